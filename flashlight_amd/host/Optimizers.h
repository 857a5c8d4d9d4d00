// First-order optimizers over the host layer's Variables: the interface of
// flashlight/fl/optim/Optimizers.h:25-75 and fl::SGDOptimizer (optim/SGDOptimizer.{h,cpp}): stochastic gradient
// descent with weight decay, momentum and Nesterov momentum, and fl::AdamOptimizer; the update of every parameter tensor
// of a step in one launch per 48 / 32 tensors (flhip_sgd_many, flhip_adam_many) instead of several tensor expressions per
// parameter.
#pragma once

#include <string>
#include <vector>

#include "Functions.h"

namespace fl {

class FirstOrderOptimizer {
 public:
  FirstOrderOptimizer(const std::vector<Variable>& parameters, double learningRate)
      : parameters_(parameters), lr_(learningRate) {}
  virtual ~FirstOrderOptimizer() = default;
  virtual void step() = 0;
  double getLr() const { return lr_; }
  void setLr(double lr) { lr_ = lr; }
  virtual void zeroGrad();
  virtual std::string prettyString() const = 0;

 protected:
  std::vector<Variable> parameters_;
  double lr_;
};

class SGDOptimizer : public FirstOrderOptimizer {
 public:
  SGDOptimizer(const std::vector<Variable>& parameters, float learningRate, float momentum = 0, float weightDecay = 0,
               bool useNesterov = false);
  // parameters without a gradient are left alone (SGDOptimizer.cpp:40-42); the others are updated in place
  void step() override;
  std::string prettyString() const override;

 private:
  bool useNesterov_;
  float mu_, wd_;
  std::vector<Tensor> velocities_;
};

// fl::AdamOptimizer (optim/AdamOptimizer.{h,cpp}): Adam with decoupled weight decay and the bias-corrected rate
class AdamOptimizer : public FirstOrderOptimizer {
 public:
  AdamOptimizer(const std::vector<Variable>& parameters, float learningRate, float beta1 = 0.9f, float beta2 = 0.999f,
                float epsilon = 1e-8f, float weightDecay = 0);
  void step() override;
  std::string prettyString() const override;

 private:
  float beta1_, beta2_, eps_, wd_;
  int count_ = 0;
  std::vector<Tensor> biasedFirst_, biasedSecond_;
};

}  // namespace fl
