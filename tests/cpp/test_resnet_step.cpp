// ResNet-50 (configs[4]: 224x224x3 input, conv / BatchNorm / max-pool forward and backward
// through the HIP extension) from the host modules and the tape, in fp32 and in bf16
// storage with fp32 master weights.
//
// What is checked.  A whole step cannot be compared with the CPU checker end to end at a
// useful bound: summation-order differences of 1e-7 grow through 53 convolutions, each
// followed by a batch norm, and through ReLU masks that flip.  So every operation of the
// real step is checked on its own instead: an observer on the host layer receives each
// operation's device inputs and outputs, runs the CPU checker on THOSE inputs and
// compares (conv2d, conv2dBackwardData, conv2dBackwardFilterBias, batchnorm,
// batchnormBackward, pool2d, pool2dBackward, relu, reluBackward, add, gradient
// accumulation, casts, linear, logSoftmax, categoricalCrossEntropy, and the fused
// batchnorm + ReLU (+ residual) pair against the checker's composition).  Bounds: relative
// L2 1e-4 for fp32 results, 2e-2 for bf16 results (the stated tolerances; the run also
// prints the worst case per operation), pooling bit for bit.
// On top: shapes, 161 parameter tensors each with a finite gradient, run-to-run bit
// identity, and the bf16 step's loss against the fp32 step's.
#include <cmath>
#include <csignal>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <execinfo.h>
#include <map>
#include <random>
#include <string>
#include <unistd.h>
#include <vector>

#include "OpObserver.h"
#include "Resnet.h"
#include "flhip.h"
#include "flref.h"

using namespace fl;

static std::vector<float> randn(size_t n, unsigned seed) {
  std::mt19937 gen(seed);
  std::normal_distribution<float> d(0.f, 1.f);
  std::vector<float> v(n);
  for (auto& x : v) x = d(gen);
  return v;
}
static double relL2(const std::vector<float>& a, const std::vector<float>& b) {
  if (a.size() != b.size()) return 1e30;
  double num = 0, den = 0;
  for (size_t i = 0; i < a.size(); ++i) {
    num += ((double)a[i] - b[i]) * ((double)a[i] - b[i]);
    den += (double)b[i] * b[i];
  }
  return den > 0 ? std::sqrt(num / den) : std::sqrt(num);
}
static std::vector<float> host(const Tensor& t) { return t.toHostVector(); }
static std::vector<float> toBf16(std::vector<float> v) {
  for (auto& f : v) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) <= 0x7f800000u) u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    std::memcpy(&f, &u, 4);
  }
  return v;
}

// Replays each observed operation on the CPU checker.
class OracleChecker : public detail::OpObserver {
 public:
  struct Stat {
    long calls = 0, failed = 0;
    double worst = 0;
  };
  std::map<std::string, Stat> stats;
  bool active = true;

  void end(const detail::OpEvent& e) override {
    if (!active) return;
    active = false;   // the copies to the host below cast bf16 tensors: do not observe those casts
    try {
      check(e);
    } catch (...) {
      active = true;
      throw;
    }
    active = true;
  }

 private:
  // result `got` of type `t` against the checker's fp32 `ref`; a bf16 result is compared with the
  // checker's value as it is (the rounding is part of the 2e-2 allowance)
  void cmp(const std::string& what, const Tensor& got, const std::vector<float>& ref) {
    const double tol = got.type() == dtype::bf16 ? 2e-2 : 1e-4;
    const double e = relL2(host(got), ref);
    Stat& s = stats[what + (got.type() == dtype::bf16 ? " [bf16]" : " [f32]")];
    s.calls++;
    if (!(e <= tol)) {
      s.failed++;
      if (s.failed <= 3) std::printf("  FAILED %s: relative L2 %.3e > %.0e (%zu elements)\n", what.c_str(), e, tol, ref.size());
    }
    if (e > s.worst || !(e == e)) s.worst = e;
  }
  void same(const std::string& what, const std::vector<float>& got, const std::vector<float>& ref) {
    Stat& s = stats[what + " [exact]"];
    s.calls++;
    if (got != ref) {
      s.failed++;
      s.worst = 1;
      if (s.failed <= 3) std::printf("  FAILED %s: not bit-identical\n", what.c_str());
    }
  }
  static flref_conv convGeom(const Shape& in, const Shape& w, const std::vector<long long>& a) {
    flref_conv d{};
    d.W = (int)in.dim(0); d.H = (int)in.dim(1); d.C = (int)in.dim(2); d.N = (int)in.dim(3);
    d.KW = (int)w.dim(0); d.KH = (int)w.dim(1); d.K = (int)w.dim(3);
    d.sx = (int)a[0]; d.sy = (int)a[1]; d.px = (int)a[2]; d.py = (int)a[3]; d.dil_x = (int)a[4]; d.dil_y = (int)a[5];
    d.groups = (int)a[6];
    return d;
  }
  static flref_pool poolGeom(const Shape& in, const std::vector<long long>& a) {
    flref_pool d{};
    d.W = (int)in.dim(0); d.H = (int)in.dim(1); d.C = (int)in.dim(2); d.N = (int)in.dim(3);
    d.wx = (int)a[0]; d.wy = (int)a[1]; d.sx = (int)a[2]; d.sy = (int)a[3]; d.px = (int)a[4]; d.py = (int)a[5];
    d.mode = (int)a[6];
    return d;
  }
  static std::vector<uint8_t> bytes(const Tensor& t) {
    std::vector<uint8_t> v((size_t)t.elements());
    t.toHost(v.data());
    return v;
  }
  static std::vector<float> varOf(const std::vector<float>& invstd, double eps) {
    std::vector<float> v(invstd.size());
    for (size_t i = 0; i < v.size(); ++i) v[i] = (float)(1.0 / ((double)invstd[i] * invstd[i]) - eps);
    return v;
  }

  void check(const detail::OpEvent& e) {
    const std::string op = e.op;
    const auto& in = e.inputs;
    const auto& out = e.outputs;
    if (op == "conv2d") {
      const flref_conv d = convGeom(in[0].shape(), in[1].shape(), e.ints);
      const auto x = host(in[0]), w = host(in[1]), b = host(in[2]);
      std::vector<float> y((size_t)out[0].elements());
      flref_conv2d_fwd(&d, x.data(), w.data(), b.empty() ? nullptr : b.data(), y.data());
      cmp(op, out[0], y);
    } else if (op == "conv2dBackwardData") {
      const flref_conv d = convGeom(out[0].shape(), in[1].shape(), e.ints);
      const auto dy = host(in[0]), w = host(in[1]);
      std::vector<float> dx((size_t)out[0].elements());
      flref_conv2d_bwd_data(&d, dy.data(), w.data(), dx.data());
      cmp(op, out[0], dx);
    } else if (op == "conv2dBackwardDataAdd") {
      // the pass's result and the gradient the input already held, each in the storage type, summed
      const flref_conv d = convGeom(out[0].shape(), in[1].shape(), e.ints);
      const auto dy = host(in[0]), w = host(in[1]), add = host(in[2]);
      std::vector<float> dx((size_t)out[0].elements());
      flref_conv2d_bwd_data(&d, dy.data(), w.data(), dx.data());
      for (size_t i = 0; i < dx.size(); ++i) dx[i] += add[i];
      cmp(op, out[0], dx);
    } else if (op == "conv2dBackwardFilterBias") {
      const flref_conv d = convGeom(in[1].shape(), out[0].shape(), e.ints);
      const auto dy = host(in[0]), x = host(in[1]);
      std::vector<float> dw((size_t)out[0].elements()), db((size_t)d.K);
      flref_conv2d_bwd_filter(&d, x.data(), dy.data(), dw.data(), db.data());
      cmp(op + " dw", out[0], dw);
      if (!out[1].isEmpty()) cmp(op + " db", out[1], db);
    } else if (op == "pool2d") {
      const flref_pool d = poolGeom(in[0].shape(), e.ints);
      const auto x = host(in[0]);
      std::vector<float> y((size_t)out[0].elements());
      std::vector<uint8_t> am(d.mode == 0 ? y.size() : 0);
      flref_pool2d_fwd(&d, x.data(), y.data(), am.empty() ? nullptr : am.data());
      // max pooling selects; averages of bf16 values round once
      if (d.mode == 0) {
        same(op + " values", host(out[0]), y);
        if (!out[1].isEmpty()) {
          Stat& s = stats[op + " argmax [exact]"];
          s.calls++;
          if (bytes(out[1]) != am) { s.failed++; s.worst = 1; std::printf("  FAILED pool2d argmax bytes\n"); }
        }
      } else if (out[0].type() == dtype::f32) {
        same(op + " avg", host(out[0]), y);
      } else {
        cmp(op + " avg", out[0], y);
      }
    } else if (op == "pool2dBackward") {
      const flref_pool d = poolGeom(out[0].shape(), e.ints);
      const auto dy = host(in[0]);
      std::vector<uint8_t> am = in[1].isEmpty() ? std::vector<uint8_t>() : bytes(in[1]);
      std::vector<float> dx((size_t)out[0].elements());
      flref_pool2d_bwd(&d, dy.data(), am.empty() ? nullptr : am.data(), dx.data());
      if (out[0].type() == dtype::f32) same(op, host(out[0]), dx);
      else cmp(op, out[0], dx);
    } else if (op == "batchnorm" || op == "batchnormRelu") {
      // inputs {x, gamma, beta, runMean, runVar[, residual]}, outputs {y, saveMean, saveInvStd}
      const long long outer = e.ints[0], C = e.ints[1], inner = e.ints[2];
      if (!e.ints[3]) return;   // inference mode is not part of a training step
      const auto x = host(in[0]), g = host(in[1]), b = host(in[2]);
      std::vector<float> y(x.size()), mean((size_t)C), var((size_t)C);
      flref_bn_fwd_train(outer, C, inner, x.data(), g.empty() ? nullptr : g.data(), b.empty() ? nullptr : b.data(),
                         e.reals[1], y.data(), mean.data(), var.data());
      if (op == "batchnormRelu") {
        if (in.size() > 5 && !in[5].isEmpty()) {
          const auto r = host(in[5]);
          for (size_t i = 0; i < y.size(); ++i) y[i] += r[i];
        }
        std::vector<float> z(y.size());
        flref_relu_fwd((int64_t)y.size(), y.data(), z.data());
        y.swap(z);
      }
      cmp(op + " y", out[0], y);
      cmp(op + " mean", out[1], mean);
      std::vector<float> is((size_t)C);
      for (long long c = 0; c < C; ++c) is[(size_t)c] = (float)(1.0 / std::sqrt((double)var[(size_t)c] + e.reals[1]));
      cmp(op + " invstd", out[2], is);
    } else if (op == "batchnormBackward" || op == "batchnormReluBackward") {
      // inputs {dy, x, gamma, saveMean, saveInvStd[, y]}, outputs {dx, dgamma, dbeta[, dresidual]}
      const long long outer = e.ints[0], C = e.ints[1], inner = e.ints[2];
      auto dy = host(in[0]);
      const auto x = host(in[1]), g = host(in[2]), mean = host(in[3]), is = host(in[4]);
      if (op == "batchnormReluBackward") {
        const auto y = host(in[5]);
        std::vector<float> dz(dy.size());
        flref_relu_bwd((int64_t)dy.size(), dy.data(), y.data(), dz.data());
        dy.swap(dz);
        // the masked gradient is what the shortcut branch receives, in the storage type
        if (out.size() > 3 && !out[3].isEmpty()) same(op + " dresidual", host(out[3]), dy);
      }
      // saveInvStd -> the variance the checker takes; eps cancels out again inside it
      const double eps = 1e-5;
      const auto var = varOf(is, eps);
      std::vector<float> dx(x.size()), dg((size_t)C), db((size_t)C);
      flref_bn_bwd(outer, C, inner, x.data(), dy.data(), g.empty() ? nullptr : g.data(), mean.data(), var.data(), eps,
                   dx.data(), dg.data(), db.data());
      cmp(op + " dx", out[0], dx);
      cmp(op + " dgamma", out[1], dg);
      cmp(op + " dbeta", out[2], db);
    } else if (op == "relu") {
      const auto x = host(in[0]);
      std::vector<float> y(x.size());
      flref_relu_fwd((int64_t)x.size(), x.data(), y.data());
      same(op, host(out[0]), y);
    } else if (op == "reluBackward") {
      const auto dy = host(in[0]), x = host(in[1]);
      std::vector<float> dx(x.size());
      flref_relu_bwd((int64_t)x.size(), dy.data(), x.data(), dx.data());
      same(op, host(out[0]), dx);
    } else if (op == "add" || op == "addGrad") {
      const auto a = host(in[0]), b = host(in[1]);
      std::vector<float> c(a.size());
      for (size_t i = 0; i < a.size(); ++i) c[i] = a[i] + b[i];
      // one fp32 addition, rounded once to the storage type: exact in both
      same(op, host(out[0]), out[0].type() == dtype::bf16 ? toBf16(c) : c);
    } else if (op == "astype") {
      // one conversion or several in one launch: inputs[i] -> outputs[i]
      for (size_t i = 0; i < in.size() && i < out.size(); ++i) {
        const auto a = host(in[i]);
        same(op, host(out[i]), out[i].type() == dtype::bf16 ? toBf16(a) : a);
      }
    } else if (op == "linear") {
      const int M = (int)e.ints[0], K = (int)e.ints[1], N = (int)e.ints[2];
      const auto x = host(in[0]), w = host(in[1]), b = host(in[2]);
      std::vector<float> y((size_t)M * N);
      flref_matmul(M, N, K, 0, 0, w.data(), x.data(), b.empty() ? nullptr : b.data(), y.data());
      cmp(op, out[0], y);
    } else if (op == "linearBackward") {
      const int M = (int)e.ints[0], K = (int)e.ints[1], N = (int)e.ints[2];
      const auto g = host(in[0]), x = host(in[1]), w = host(in[2]);
      if (!out[0].isEmpty()) {
        std::vector<float> dx((size_t)K * N);
        flref_matmul(K, N, M, 1, 0, w.data(), g.data(), nullptr, dx.data());
        cmp(op + " dx", out[0], dx);
      }
      if (!out[1].isEmpty()) {
        std::vector<float> dw((size_t)M * K);
        flref_matmul(M, K, N, 0, 1, g.data(), x.data(), nullptr, dw.data());
        cmp(op + " dw", out[1], dw);
      }
      if (!out[2].isEmpty()) {
        std::vector<float> db((size_t)M);
        flref_sum_columns(M, N, g.data(), db.data());
        cmp(op + " db", out[2], db);
      }
    } else if (op == "logSoftmax") {
      const auto x = host(in[0]);
      std::vector<float> y(x.size());
      flref_logsoftmax_fwd((int)e.ints[0], (int)e.ints[1], x.data(), y.data());
      cmp(op, out[0], y);
    } else if (op == "logSoftmaxBackward") {
      const auto dy = host(in[0]), y = host(in[1]);
      std::vector<float> dx(y.size());
      flref_logsoftmax_bwd((int)e.ints[0], (int)e.ints[1], dy.data(), y.data(), dx.data());
      cmp(op, out[0], dx);
    } else if (op == "categoricalCrossEntropy") {
      const int C = (int)e.ints[0], X = (int)e.ints[1];
      const auto lp = host(in[0]);
      std::vector<int32_t> tg((size_t)X);
      in[1].toHost(tg.data());
      float loss[2], count;
      flref_cce_fwd(C, X, lp.data(), tg.data(), (int)e.ints[3], nullptr, loss, &count);
      if (e.ints[2] != 0) cmp(op, out[0], {e.ints[2] == 1 ? loss[1] : loss[0]});
    } else if (op == "categoricalCrossEntropyBackward") {
      const int C = (int)e.ints[0], X = (int)e.ints[1];
      const auto g = host(in[0]), st = host(in[2]);
      std::vector<int32_t> tg((size_t)X);
      in[1].toHost(tg.data());
      std::vector<float> dx((size_t)C * X);
      flref_cce_bwd(C, X, g.data(), tg.data(), (int)e.ints[3], (int)e.ints[2], st[1], dx.data());
      cmp(op, out[0], dx);
    } else {
      stats[std::string("(unchecked) ") + op].calls++;
    }
  }
};

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
    int fail = 0;
    float lossOf[3] = {0, 0, 0};
    // fp32 and bf16 with BatchNorm -> (+ shortcut) -> ReLU fused (the default), then bf16 with the
    // three reference operators composed
    for (int pass = 0; pass < 3; ++pass) {
      const bool half = pass >= 1;
      pkg::vision::setFusedBatchNormRelu(pass < 2);
      detail::setFusedGradAdd(pass < 2);
      setSeed(3);
      auto model = pkg::vision::resnet50();
      const auto params = model->params();
      std::printf("ResNet-50, %s, %s, batch %d: %zu parameter tensors\n", half ? "bf16 storage" : "fp32",
                  pass < 2 ? "fused batch norm + ReLU" : "composed operators", B, params.size());
      Tensor x = Tensor::fromVector({224, 224, 3, B}, randn((size_t)B * 3 * 224 * 224, 1));
      Variable in(half ? x.astype(dtype::bf16) : x, false);
      std::vector<int32_t> labels(B);
      for (int i = 0; i < B; ++i) labels[i] = (i * 37 + 11) % 1000;
      Variable target(Tensor::fromHost(Shape({B}), dtype::s32, labels.data()), false);

      Variable logits = model->forward(in);
      if (!(logits.shape() == Shape({1000, B}))) { std::printf("FAILED: output shape %s\n", logits.shape().toString().c_str()); ++fail; }
      if (params.size() != 161) { std::printf("FAILED: %zu parameter tensors, expected 161\n", params.size()); ++fail; }

      auto run = [&]() {
        StepResult r;
        r.loss = step(*model, in, target).tensor().toHostVector()[0];
        for (size_t i : {size_t(0), size_t(1), params.size() / 2, params.size() - 2, params.size() - 1})
          r.grads.push_back(model->param((int)i).grad().tensor().toHostVector());
        return r;
      };
      // the checked step: every operation against the CPU checker on its own inputs
      OracleChecker checker;
      detail::setOpObserver(&checker);
      const StepResult a = run();
      detail::setOpObserver(nullptr);
      long ops = 0;
      for (const auto& kv : checker.stats) {
        std::printf("  %-44s %5ld calls, worst relative L2 %.2e%s\n", kv.first.c_str(), kv.second.calls, kv.second.worst,
                    kv.second.failed ? "  FAILED" : "");
        fail += (int)kv.second.failed;
        if (kv.first.rfind("(unchecked)", 0) == 0) { std::printf("FAILED: operation without a check\n"); ++fail; }
        ops += kv.second.calls;
      }
      std::printf("  %ld results checked against the CPU checker\n", ops);
      for (const char* need : {"conv2d", "conv2dBackwardData", "conv2dBackwardFilterBias dw", "pool2d values", "pool2dBackward",
                               pass < 2 ? "batchnormRelu y" : "batchnorm y", pass < 2 ? "batchnormReluBackward dx" : "relu",
                               pass < 2 ? "conv2dBackwardDataAdd" : "addGrad"}) {
        bool seen = false;
        for (const auto& kv : checker.stats) seen = seen || kv.first.rfind(need, 0) == 0;
        if (!seen) { std::printf("FAILED: no %s in the step\n", need); ++fail; }
      }
      for (const auto& p : model->params())
        if (!p.isGradAvailable()) { std::printf("FAILED: parameter without gradient\n"); ++fail; break; }
      for (const auto& g : a.grads)
        for (float v : g)
          if (!std::isfinite(v)) { std::printf("FAILED: non-finite gradient\n"); ++fail; break; }
      const StepResult a2 = run();          // the kernels are deterministic: bit-identical
      if (a.loss != a2.loss) { std::printf("FAILED: run-to-run difference in the loss\n"); ++fail; }
      for (size_t i = 0; i < a.grads.size(); ++i)
        if (a.grads[i] != a2.grads[i]) { std::printf("FAILED: run-to-run difference in gradient %zu\n", i); ++fail; }
      std::printf("  loss %.6f\n", a.loss);
      if (!std::isfinite(a.loss)) { std::printf("FAILED: loss\n"); ++fail; }
      lossOf[pass] = a.loss;
    }
    // same weights, same input up to bf16 rounding: the losses agree to the bf16 bound
    for (int pass = 1; pass < 3; ++pass)
      if (std::fabs(lossOf[0] - lossOf[pass]) > 2e-2f * std::fabs(lossOf[0])) {
        std::printf("FAILED: bf16 loss %.6f against fp32 loss %.6f\n", lossOf[pass], lossOf[0]);
        ++fail;
      }
    pkg::vision::setFusedBatchNormRelu(true);
    detail::setFusedGradAdd(true);
    std::printf(fail ? "%d check(s) FAILED\n" : "ResNet-50 step checks passed\n", fail);
    std::fflush(stdout);
    return fail ? 1 : 0;
  } catch (const std::exception& e) {
    std::printf("unexpected exception: %s\n", e.what());
    return 2;
  }
}
