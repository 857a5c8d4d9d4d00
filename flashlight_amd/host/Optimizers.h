// First-order optimizers over the host layer's Variables: the interface of
// flashlight/fl/optim/Optimizers.h:25-75 and fl::SGDOptimizer (optim/SGDOptimizer.{h,cpp}): stochastic gradient
// descent with weight decay, momentum and Nesterov momentum, the update of every parameter tensor of a step in one
// launch per 48 tensors (flhip_sgd_many) instead of five tensor expressions per parameter.
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

}  // namespace fl
