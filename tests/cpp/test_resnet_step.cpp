// ResNet-50 (configs[4]) forward + backward through the host modules and the tape on the
// device.  Without arguments: batch 2, checks shapes, that every parameter receives a
// finite gradient, and that the whole step agrees between the matrix-core convolution
// kernels and the direct (one thread per result) kernels, which share no code with them.
// With arguments `<batch> <steps>`: times the step (forward, loss, backward).
#include <chrono>
#include <cmath>
#include <csignal>
#include <execinfo.h>
#include <unistd.h>

#include "flhip.h"
#include <cstdio>
#include <cstdlib>
#include <string>
#include <random>
#include <vector>

#include "Resnet.h"

using namespace fl;

static std::vector<float> randn(size_t n, unsigned seed) {
  std::mt19937 gen(seed);
  std::normal_distribution<float> d(0.f, 1.f);
  std::vector<float> v(n);
  for (auto& x : v) x = d(gen);
  return v;
}
static double relL2(const std::vector<float>& a, const std::vector<float>& b) {
  double num = 0, den = 0;
  for (size_t i = 0; i < a.size(); ++i) {
    num += ((double)a[i] - b[i]) * ((double)a[i] - b[i]);
    den += (double)b[i] * b[i];
  }
  return den > 0 ? std::sqrt(num / den) : std::sqrt(num);
}

struct StepResult {
  float loss;
  std::vector<std::vector<float>> grads;   // of a few parameters
};

static Variable step(Sequential& model, const Variable& in, const Variable& target) {
  model.zeroGrad();
  Variable out = logSoftmax(model.forward(in), 0);
  Variable loss = categoricalCrossEntropy(out, target);
  loss.backward(Variable(Tensor::fromVector({1}, {1.f}), false));
  return loss;
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

int main(int argc, char** argv) {
  std::setvbuf(stdout, nullptr, _IONBF, 0);
  std::signal(SIGSEGV, onCrash);
  std::signal(SIGBUS, onCrash);
  try {
    const int B = argc > 1 ? std::atoi(argv[1]) : 2;
    const int steps = argc > 2 ? std::atoi(argv[2]) : 0;
    setSeed(3);
    auto model = pkg::vision::resnet50();
    const auto params = model->params();
    std::printf("ResNet-50: %zu parameter tensors, batch %d\n", params.size(), B);
    Variable in(Tensor::fromVector({224, 224, 3, B}, randn((size_t)B * 3 * 224 * 224, 1)), false);
    std::vector<int32_t> labels(B);
    for (int i = 0; i < B; ++i) labels[i] = (i * 37 + 11) % 1000;
    Variable target(Tensor::fromHost(Shape({B}), dtype::s32, labels.data()), false);

    if (steps > 0) {
      // "bf16" as third argument: bf16 activations, parameters cast per call by the modules
      // (fp32 master copies, fp32 batch-norm parameters and statistics)
      const bool half = argc > 3 && std::string(argv[3]) == "bf16";
      if (half) in = Variable(in.tensor().astype(dtype::bf16), false);
      for (int i = 0; i < 3; ++i) step(*model, in, target);
      fl::sync();
      const auto t0 = std::chrono::steady_clock::now();
      float last = 0.f;
      for (int i = 0; i < steps; ++i) last = step(*model, in, target).tensor().toHostVector()[0];
      fl::sync();
      const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / steps;
      std::printf("forward + loss + backward (%s): %.2f ms per step (batch %d, %.1f images/s), loss %.4f, "
                  "device cache %.1f MB\n", half ? "bf16" : "f32", ms, B, B / ms * 1e3, last, deviceCacheBytes() / 1e6);
      std::fflush(stdout);
      // timing mode leaves through exit() so that a profiler's exit handlers run
      std::exit(0);
    }

    int fail = 0;
    auto run = [&](const char* algo) {
      if (flhip_set_option("CONV_ALGO", algo) != FLHIP_OK) throw std::runtime_error(flhip_last_error());
      StepResult r;
      r.loss = step(*model, in, target).tensor().toHostVector()[0];
      for (size_t i : {size_t(0), size_t(1), params.size() / 2, params.size() - 2, params.size() - 1})
        r.grads.push_back(model->param((int)i).grad().tensor().toHostVector());
      return r;
    };
    Variable logits = model->forward(in);
    if (!(logits.shape() == Shape({1000, B}))) { std::printf("FAILED: output shape %s\n", logits.shape().toString().c_str()); ++fail; }
    if (params.size() != 161) { std::printf("FAILED: %zu parameter tensors, expected 161\n", params.size()); ++fail; }
    const StepResult a = run(nullptr);
    for (const auto& p : model->params()) {
      if (!p.isGradAvailable()) { std::printf("FAILED: parameter without gradient\n"); ++fail; break; }
    }
    const StepResult a2 = run(nullptr);          // the kernels are deterministic: bit-identical
    const StepResult b = run("direct");
    const StepResult g = run("gather");          // matrix cores again, another summation order
    flhip_set_option("CONV_ALGO", nullptr);
    std::printf("loss %.6f (default) %.6f (direct kernels) %.6f (gather kernels)\n", a.loss, b.loss, g.loss);
    if (!std::isfinite(a.loss) || std::fabs(a.loss - b.loss) > 1e-4f * std::fabs(b.loss)) { std::printf("FAILED: loss\n"); ++fail; }
    // The step is a chain of 53 convolutions, each followed by a batch norm, and of ReLU
    // masks: summation-order differences of 1e-7 grow on the way back to the first layers.
    // The gather kernels add in the direct kernels' order and reproduce them to 4e-7; every
    // kernel family with another order (FLHIP_CONV_SKIP leaves families out one at a time)
    // lands 1.5-2.5 % away at the first layer, at batch 2 and at batch 8 alike, while the
    // last layers agree to 1e-5.  The per-layer parity tests carry the tight bounds; here
    // the bound only catches gross errors.
    for (size_t i = 0; i < a.grads.size(); ++i) {
      const double e = relL2(a.grads[i], b.grads[i]), eg = relL2(g.grads[i], b.grads[i]);
      std::printf("  gradient %zu: %zu elements, relative L2 difference to direct: default %.2e, gather %.2e\n", i,
                  a.grads[i].size(), e, eg);
      if (a.grads[i] != a2.grads[i]) { std::printf("FAILED: run-to-run difference in gradient %zu\n", i); ++fail; }
      const double tol = i + 2 >= a.grads.size() ? 1e-4 : 6e-2;
      if (!(e <= tol)) { std::printf("FAILED: gradient %zu\n", i); ++fail; }
    }
    std::printf(fail ? "%d check(s) FAILED\n" : "ResNet-50 step checks passed\n", fail);
    std::fflush(stdout);
    return fail ? 1 : 0;
  } catch (const std::exception& e) {
    std::printf("unexpected exception: %s\n", e.what());
    return 2;
  }
}
