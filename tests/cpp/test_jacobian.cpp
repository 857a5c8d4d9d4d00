// The reference's autograd tests for the operators of the extension, restated on this
// host layer: forward Jacobian by central differences against the Jacobian the tape
// returns (flashlight/fl/test/autograd/AutogradTestUtils.h:32-70, allClose = largest
// absolute difference below `precision`), with the shapes, arguments and tolerances of
//   AutogradConv2DTest.cpp:21-74 (Convolve), :137-162 (ConvolveFilterGroups),
//     :164-213 (ConvolveDilation)
//   AutogradTest.cpp:333-337 (Pooling)
//   AutogradNormalizationTest.cpp:228-256 (BatchNormJacobian), :294-324
//     (BatchNormJacobianMultipleAxes), :365-383 (LayerNormJacobian)
//   AutogradRnnTest.cpp:24-160 (rnn: input, weights, initial states, through y and hy);
//     the reference runs these in f64, this backend is f32, hence a larger
//     perturbation and tolerance there.
// Everything runs through the device library; nothing here uses the CPU checker.

#include <cmath>
#include <cstdio>
#include <functional>
#include <random>
#include <string>
#include <vector>

#include "Functions.h"
#include "HipAutogradExtension.h"

using namespace fl;

static int g_fail = 0;
#define CHECK(c)                                                          \
  do {                                                                    \
    if (!(c)) {                                                           \
      std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #c);        \
      ++g_fail;                                                           \
    }                                                                     \
  } while (0)

// fl::rand: uniform [0, 1)
static Variable randVar(const Shape& shape, unsigned seed, bool calcGrad) {
  std::mt19937 gen(seed);
  std::uniform_real_distribution<float> d(0.f, 1.f);
  std::vector<float> v((size_t)shape.elements());
  for (float& x : v) x = d(gen);
  return Variable(Tensor::fromVector(shape, v), calcGrad);
}

using JacobianFunc = std::function<Variable(Variable&)>;

// largest absolute difference between the two Jacobians
static double jacobianError(const JacobianFunc& func, const Variable& input, float perturbation) {
  const Shape shape = input.shape();
  std::vector<float> x = input.tensor().toHostVector();
  const size_t nin = x.size();
  Variable probe(Tensor::fromVector(shape, x), true);
  const Shape outShape = func(probe).shape();
  const size_t nout = (size_t)outShape.elements();
  std::vector<float> fwd(nout * nin), bwd(nout * nin);
  for (size_t i = 0; i < nin; ++i) {
    const float orig = x[i];
    x[i] = orig - perturbation;
    Variable a(Tensor::fromVector(shape, x), true);
    const std::vector<float> outa = func(a).tensor().toHostVector();
    x[i] = orig + perturbation;
    Variable b(Tensor::fromVector(shape, x), true);
    const std::vector<float> outb = func(b).tensor().toHostVector();
    x[i] = orig;
    for (size_t o = 0; o < nout; ++o) fwd[o * nin + i] = (outb[o] - outa[o]) * 0.5f / perturbation;
  }
  std::vector<float> dout(nout, 0.f);
  for (size_t o = 0; o < nout; ++o) {
    dout[o] = 1.f;
    Variable in(Tensor::fromVector(shape, x), true);
    Variable out = func(in);
    out.backward(Variable(Tensor::fromVector(outShape, dout), false));
    const std::vector<float> g = in.grad().tensor().toHostVector();
    for (size_t i = 0; i < nin; ++i) bwd[o * nin + i] = g[i];
    dout[o] = 0.f;
  }
  double worst = 0;
  for (size_t k = 0; k < fwd.size(); ++k) {
    const double d = std::fabs((double)fwd[k] - bwd[k]);
    if (!(d <= worst)) worst = d;   // NaN propagates
  }
  return worst;
}

static bool jacobianTest(const char* what, const JacobianFunc& func, const Variable& input, float precision = 1e-5f,
                         float perturbation = 1e-4f) {
  const double err = jacobianError(func, input, perturbation);
  std::printf("  %-44s max |fd - tape| = %.3g (limit %.3g)\n", what, err, precision);
  std::fflush(stdout);
  return err < precision;
}

static void convCase(const char* name, int groups, int dx, int dy, float tolIn, float tolWt, float tolBs, bool biasInAll) {
  std::printf("%s\n", name);
  const int channel = 8;
  Variable in = randVar({10, 9, channel, 7}, 1, true);
  Variable wt = randVar({4, 3, channel / groups, 6}, 2, true);
  Variable bs = randVar({1, 1, 6, 1}, 3, true);
  const int px = 2, py = 1, sx = 1, sy = 1;
  CHECK(jacobianTest("input", [&](Variable& input) {
    return biasInAll ? conv2d(input, wt, bs, sx, sy, px, py, dx, dy, groups) : conv2d(input, wt, sx, sy, px, py, dx, dy, groups);
  }, in, tolIn));
  CHECK(jacobianTest("weights", [&](Variable& weight) {
    return biasInAll ? conv2d(in, weight, bs, sx, sy, px, py, dx, dy, groups) : conv2d(in, weight, sx, sy, px, py, dx, dy, groups);
  }, wt, tolWt));
  CHECK(jacobianTest("bias", [&](Variable& bias) { return conv2d(in, wt, bias, sx, sy, px, py, dx, dy, groups); }, bs, tolBs));
}

static void testPooling() {
  std::printf("Pooling\n");
  Variable in = randVar({3, 3, 1, 1}, 4, true);
  CHECK(jacobianTest("max 2x2 stride 1", [&](Variable& input) { return pool2d(input, 2, 2, 1, 1); }, in, 1e-3f));
  CHECK(jacobianTest("avg 2x2 stride 1", [&](Variable& input) {
    return pool2d(input, 2, 2, 1, 1, 0, 0, PoolingMode::AVG_INCLUDE_PADDING);
  }, in, 1e-3f));
}

static void bnCase(const char* name, const Shape& shape, const std::vector<int>& featAxes, float precision, float perturbation,
                   bool paramsToo) {
  std::printf("%s\n", name);
  Variable input = randVar(shape, 5, true);
  Dim nfeatures = 1;
  for (int ax : featAxes) nfeatures *= input.dim(ax);
  Variable runningMean = randVar({nfeatures}, 6, false), runningVar = randVar({nfeatures}, 7, false);
  Variable weight = randVar({nfeatures}, 8, true), bias = randVar({nfeatures}, 9, true);
  CHECK(jacobianTest("input", [&](Variable& in) {
    return batchnorm(in, weight, bias, runningMean, runningVar, featAxes, true, 0.0, 1e-5);
  }, input, precision, perturbation));
  if (!paramsToo) return;
  CHECK(jacobianTest("weight", [&](Variable& wt) {
    return batchnorm(input, wt, bias, runningMean, runningVar, featAxes, true, 0.0, 1e-5);
  }, weight, precision, perturbation));
  CHECK(jacobianTest("bias", [&](Variable& bs) {
    return batchnorm(input, weight, bs, runningMean, runningVar, featAxes, true, 0.0, 1e-5);
  }, bias, precision, perturbation));
}

static void rnnCase(const char* name, RnnMode mode, size_t nParams) {
  std::printf("%s\n", name);
  const int numLayers = 2, hiddenSize = 2, inputSize = 2, batchSize = 2, seqLength = 3;
  const bool bidirectional = true;
  const float precision = 2e-3f, perturbation = 1e-2f;
  Variable in = randVar({inputSize, batchSize, seqLength}, 10, true);
  Variable w = randVar({(Dim)nParams}, 11, true);
  const Variable none;
  CHECK(jacobianTest("y wrt input", [&](Variable& input) {
    return std::get<0>(rnn(input, none, none, w, hiddenSize, numLayers, mode, bidirectional, 0.0f));
  }, in, precision, perturbation));
  CHECK(jacobianTest("y wrt weights", [&](Variable& weights) {
    return std::get<0>(rnn(in, none, none, weights, hiddenSize, numLayers, mode, bidirectional, 0.0f));
  }, w, precision, perturbation));
  Variable hx = randVar({hiddenSize, batchSize, numLayers * 2}, 12, true);
  CHECK(jacobianTest("y wrt hx", [&](Variable& hiddenState) {
    return std::get<0>(rnn(in, hiddenState, none, w, hiddenSize, numLayers, mode, bidirectional, 0.0f));
  }, hx, precision, perturbation));
  CHECK(jacobianTest("hy wrt input", [&](Variable& input) {
    return std::get<1>(rnn(input, none, none, w, hiddenSize, numLayers, mode, bidirectional, 0.0f));
  }, in, precision, perturbation));
  if (mode == RnnMode::LSTM) {
    Variable cx = randVar({hiddenSize, batchSize, numLayers * 2}, 13, true);
    CHECK(jacobianTest("y wrt cx", [&](Variable& cellState) {
      return std::get<0>(rnn(in, hx, cellState, w, hiddenSize, numLayers, mode, bidirectional, 0.0f));
    }, cx, precision, perturbation));
    CHECK(jacobianTest("cy wrt input", [&](Variable& input) {
      return std::get<2>(rnn(input, none, none, w, hiddenSize, numLayers, mode, bidirectional, 0.0f));
    }, in, precision, perturbation));
  }
}

int main() {
  setvbuf(stdout, nullptr, _IONBF, 0);
  try {
    convCase("Convolve", 1, 1, 1, 0.06f, 0.06f, 0.03f, false);
    convCase("ConvolveFilterGroups", 2, 1, 1, 0.06f, 0.05f, 0.02f, true);
    convCase("ConvolveDilation", 1, 2, 1, 0.06f, 0.05f, 0.02f, true);
    testPooling();
    bnCase("BatchNormJacobian", {8, 8, 3, 16}, {2}, 1e-2f, 1e-4f, true);
    bnCase("BatchNormJacobianMultipleAxes", {8, 8, 3, 16}, {0, 1, 2}, 1e-2f, 1e-3f, true);
    bnCase("LayerNormJacobian", {7, 7, 3, 10}, {0, 1, 2, 3}, 1e-2f, 1e-4f, false);
    rnnCase("rnn TANH", RnnMode::TANH, 56);
    rnnCase("rnn LSTM", RnnMode::LSTM, 224);
    rnnCase("rnn GRU", RnnMode::GRU, 168);
    fl::sync();
  } catch (const std::exception& e) {
    std::printf("unexpected exception: %s\n", e.what());
    return 2;
  }
  std::printf(g_fail ? "%d check(s) FAILED\n" : "all Jacobian checks passed\n", g_fail);
  std::fflush(stdout);
  return g_fail ? 1 : 0;
}
