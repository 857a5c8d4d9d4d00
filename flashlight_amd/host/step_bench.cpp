// Whole training steps through the host layer, timed: the ResNet-50 step of configs[4]
// (224x224x3, forward + logSoftmax / categoricalCrossEntropy + backward) and the speech
// stack of configs[3] (three 21x1 convolutions, each with batch norm and ReLU, forward +
// backward).  Prints one JSON object: wall time per step and, from a second, instrumented
// run, the device time per operation class (HIP events around every operation of the
// host layer) with the idle gaps between operations.
//
// usage: flhip_step_bench resnet50|speech [batch] [steps] [warmup] [f32|bf16|f16] [unfused|fused] [sgd]
// ("unfused": BatchNorm, residual add and ReLU as three operations, the reference's composition; "sgd": the step ends
// with fl::SGDOptimizer::step - momentum 0.9, weight decay 1e-4 - on the ResNet's parameters)
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <string>
#include <vector>

#include "OpObserver.h"
#include "Optimizers.h"
#include "Resnet.h"

using namespace fl;

namespace {
std::vector<float> randn(size_t n, unsigned seed) {
  std::mt19937 gen(seed);
  std::normal_distribution<float> d(0.f, 1.f);
  std::vector<float> v(n);
  for (auto& x : v) x = d(gen);
  return v;
}

// operation name -> class of the breakdown
const char* classOf(const std::string& op) {
  static const std::map<std::string, const char*> m = {
      {"conv2d", "conv_fwd"}, {"conv2dBackwardData", "conv_bwd_data"}, {"conv2dBackwardDataAdd", "conv_bwd_data"},
      {"conv2dBackwardFilterBias", "conv_bwd_filter"},
      {"batchnorm", "bn_fwd"}, {"batchnormBackward", "bn_bwd"}, {"batchnormRelu", "bn_fwd"}, {"batchnormReluBackward", "bn_bwd"},
      {"pool2d", "pool_fwd"}, {"pool2dBackward", "pool_bwd"},
      {"relu", "relu_add"}, {"reluBackward", "relu_add"}, {"add", "relu_add"}, {"addGrad", "relu_add"},
      {"astype", "casts"}, {"linear", "linear"}, {"linearBackward", "linear"},
      {"logSoftmax", "loss"}, {"logSoftmaxBackward", "loss"}, {"categoricalCrossEntropy", "loss"},
      {"categoricalCrossEntropyBackward", "loss"}, {"(gaps)", "host_gaps"}, {"(span)", "span"}};
  auto it = m.find(op);
  return it == m.end() ? "other" : it->second;
}
}  // namespace

int main(int argc, char** argv) {
  try {
    const std::string model = argc > 1 ? argv[1] : "resnet50";
    const int B = argc > 2 ? std::atoi(argv[2]) : (model == "speech" ? 16 : 64);
    const int steps = argc > 3 ? std::atoi(argv[3]) : 10;
    const int warmup = argc > 4 ? std::atoi(argv[4]) : 3;
    const std::string dname = argc > 5 ? argv[5] : "f32";
    const bool half = dname == "bf16" || dname == "f16";
    const dtype lowType = dname == "f16" ? dtype::f16 : dtype::bf16;
    const bool unfused = argc > 6 && std::string(argv[6]) == "unfused";
    const bool sgd = argc > 7 && std::string(argv[7]) == "sgd";
    pkg::vision::setFusedBatchNormRelu(!unfused);
    detail::setFusedGradAdd(!unfused);
    setSeed(3);

    // A step enqueues its work and returns the loss tensor; nothing in it waits for the device (the seed gradient is
    // filled on the device, the loss is read back once after the timed loop), so the host runs ahead of the kernels.
    std::function<Tensor()> step;
    std::shared_ptr<Sequential> net;
    std::shared_ptr<SGDOptimizer> opt;
    std::vector<Conv2D> convs;
    std::vector<BatchNorm> bns;
    Variable in, target, gradOut;
    double flop = 0;   // convolution FLOP of one step (forward + both backward passes)
    if (model == "resnet50") {
      net = pkg::vision::resnet50();
      Tensor x = Tensor::fromVector({224, 224, 3, B}, randn((size_t)B * 3 * 224 * 224, 1));
      in = Variable(half ? x.astype(lowType) : x, false);
      std::vector<int32_t> labels(B);
      std::mt19937 gen(5);
      for (int i = 0; i < B; ++i) labels[i] = (int32_t)(gen() % 1000);
      target = Variable(Tensor::fromHost(Shape({B}), dtype::s32, labels.data()), false);
      if (sgd) opt = std::make_shared<SGDOptimizer>(net->params(), 0.01f, 0.9f, 1e-4f);
      step = [&]() {
        net->zeroGrad();
        Variable out = logSoftmax(net->forward(in), 0);
        Variable loss = categoricalCrossEntropy(out, target);
        loss.backward(Variable(Tensor::full({1}, 1., dtype::f32), false));
        if (opt) opt->step();
        return loss.tensor();
      };
    } else if (model == "speech") {
      const int T = 1500, chans[4] = {80, 250, 250, 250}, strides[3] = {1, 1, 2};
      for (int l = 0; l < 3; ++l) {
        convs.emplace_back(chans[l], chans[l + 1], 21, 1, strides[l], 1, PaddingMode::SAME, PaddingMode::SAME);
        bns.emplace_back(2, chans[l + 1]);
        flop += 3.0 * 2.0 * B * chans[l + 1] * (double)(T / strides[l]) * chans[l] * 21;
      }
      Tensor x = Tensor::fromVector({T, 1, 80, B}, randn((size_t)B * 80 * T, 71));
      in = Variable(half ? x.astype(lowType) : x, true);
      Tensor g = Tensor::fromVector({T / 2, 1, 250, B}, randn((size_t)B * 250 * (T / 2), 72));
      gradOut = Variable(half ? g.astype(lowType) : g, false);
      step = [&]() {
        for (auto& c : convs) c.zeroGrad();
        for (auto& b : bns) b.zeroGrad();
        in.zeroGrad();
        Variable h = in;
        for (int l = 0; l < 3; ++l) h = unfused ? relu(bns[l](convs[l](h))) : bns[l].forwardRelu(convs[l](h));
        h.backward(gradOut);
        return Tensor();
      };
    } else {
      std::fprintf(stderr, "unknown model %s\n", model.c_str());
      return 2;
    }

    Tensor lossT;
    for (int i = 0; i < warmup; ++i) lossT = step();
    fl::sync();
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; ++i) lossT = step();
    fl::sync();
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / steps;
    const float loss = lossT.isEmpty() ? 0.f : lossT.toHostVector()[0];

    // instrumented run: device time per operation
    StepProfiler prof;
    detail::setOpObserver(&prof);
    const int psteps = steps < 5 ? steps : 5;
    for (int i = 0; i < psteps; ++i) step();
    detail::setOpObserver(nullptr);
    const auto table = prof.collect();
    std::map<std::string, StepProfiler::Entry> classes;
    for (const auto& kv : table) {
      auto& c = classes[classOf(kv.first)];
      c.ms += kv.second.ms / psteps;
      c.calls += kv.second.calls / psteps;
    }

    std::printf("{\"model\": \"%s\", \"batch\": %d, \"dtype\": \"%s\", \"fused_bn_relu\": %s, \"optimizer\": \"%s\", \"steps\": %d, \"warmup\": %d, \"ms_per_step\": %.4f, "
                "\"samples_per_s\": %.1f, \"loss\": %.5f, \"conv_gflop_per_step\": %.2f, \"device_cache_mb\": %.1f, "
                "\"breakdown_ms\": {",
                model.c_str(), B, half ? dname.c_str() : "f32", unfused ? "false" : "true", opt ? "sgd momentum 0.9 weight decay 1e-4" : "none", steps, warmup, ms, B / ms * 1e3, loss, flop / 1e9,
                deviceCacheBytes() / 1e6);
    bool first = true;
    for (const auto& kv : classes) {
      std::printf("%s\"%s\": %.4f", first ? "" : ", ", kv.first.c_str(), kv.second.ms);
      first = false;
    }
    std::printf("}, \"calls\": {");
    first = true;
    for (const auto& kv : classes) {
      std::printf("%s\"%s\": %ld", first ? "" : ", ", kv.first.c_str(), kv.second.calls);
      first = false;
    }
    std::printf("}}\n");
    std::fflush(stdout);
    return 0;
  } catch (const std::exception& e) {
    std::fprintf(stderr, "step bench failed: %s\n", e.what());
    return 2;
  }
}
