#include "Optimizers.h"

#include <map>
#include <sstream>
#include <stdexcept>

#include "flhip.h"

namespace fl {

void FirstOrderOptimizer::zeroGrad() {
  for (auto& p : parameters_) p.zeroGrad();
}

SGDOptimizer::SGDOptimizer(const std::vector<Variable>& parameters, float learningRate, float momentum,
                           float weightDecay, bool useNesterov)
    : FirstOrderOptimizer(parameters, learningRate), useNesterov_(useNesterov), mu_(momentum), wd_(weightDecay) {
  // SGDOptimizer.cpp:29-35: zero velocities of the parameters' shapes and types
  if (momentum != 0)
    for (const auto& p : parameters_) velocities_.push_back(Tensor::full(p.shape(), 0.0, p.type()));
}

void SGDOptimizer::step() {
  // one list per storage type: a launch updates tensors of one type
  struct List {
    std::vector<void*> w, v;
    std::vector<const void*> g;
    std::vector<size_t> n;
    std::vector<Tensor> keep;      // gradients cast to the parameter's type stay alive until the launch is enqueued
  };
  std::map<int, List> lists;
  for (size_t i = 0; i < parameters_.size(); ++i) {
    Variable& p = parameters_[i];
    if (!p.isGradAvailable()) continue;
    Tensor g = p.grad().tensor();
    if (g.shape().elements() != p.shape().elements())
      throw std::invalid_argument("SGDOptimizer: a gradient does not have its parameter's size");
    if (g.type() != p.type()) g = g.astype(p.type());
    const int tag = p.type() == dtype::f32 ? FLHIP_F32 : p.type() == dtype::bf16 ? FLHIP_BF16 : p.type() == dtype::f16 ? FLHIP_F16 : -1;
    if (tag < 0) throw std::invalid_argument("SGDOptimizer: parameters must be f32, bf16 or f16");
    List& l = lists[tag];
    l.w.push_back(p.tensor().device());
    l.g.push_back(g.device());
    l.v.push_back(mu_ != 0 ? velocities_[i].device() : nullptr);
    l.n.push_back((size_t)p.tensor().elements());
    l.keep.push_back(g);
  }
  for (auto& kv : lists) {
    List& l = kv.second;
    if (flhip_sgd_many(l.w.data(), l.g.data(), mu_ != 0 ? l.v.data() : nullptr, l.n.data(), (int)l.w.size(), lr_, mu_, wd_,
                       useNesterov_ ? 1 : 0, kv.first, hipBackendStream()) != FLHIP_OK)
      throw std::runtime_error(std::string("SGDOptimizer: ") + flhip_last_error());
  }
}

AdamOptimizer::AdamOptimizer(const std::vector<Variable>& parameters, float learningRate, float beta1, float beta2,
                             float epsilon, float weightDecay)
    : FirstOrderOptimizer(parameters, learningRate), beta1_(beta1), beta2_(beta2), eps_(epsilon), wd_(weightDecay) {
  for (const auto& p : parameters_) {      // AdamOptimizer.cpp:33-42
    biasedFirst_.push_back(Tensor::full(p.shape(), 0.0, p.type()));
    biasedSecond_.push_back(Tensor::full(p.shape(), 0.0, p.type()));
  }
}

void AdamOptimizer::step() {
  ++count_;                                // :46
  struct List {
    std::vector<void*> w, m, v;
    std::vector<const void*> g;
    std::vector<size_t> n;
    std::vector<Tensor> keep;
  };
  std::map<int, List> lists;
  for (size_t i = 0; i < parameters_.size(); ++i) {
    Variable& p = parameters_[i];
    if (!p.isGradAvailable()) continue;
    Tensor g = p.grad().tensor();
    if (g.shape().elements() != p.shape().elements())
      throw std::invalid_argument("AdamOptimizer: a gradient does not have its parameter's size");
    if (g.type() != p.type()) g = g.astype(p.type());
    const int tag = p.type() == dtype::f32 ? FLHIP_F32 : p.type() == dtype::bf16 ? FLHIP_BF16 : p.type() == dtype::f16 ? FLHIP_F16 : -1;
    if (tag < 0) throw std::invalid_argument("AdamOptimizer: parameters must be f32, bf16 or f16");
    List& l = lists[tag];
    l.w.push_back(p.tensor().device());
    l.g.push_back(g.device());
    l.m.push_back(biasedFirst_[i].device());
    l.v.push_back(biasedSecond_[i].device());
    l.n.push_back((size_t)p.tensor().elements());
    l.keep.push_back(g);
  }
  for (auto& kv : lists) {
    List& l = kv.second;
    if (flhip_adam_many(l.w.data(), l.g.data(), l.m.data(), l.v.data(), l.n.data(), (int)l.w.size(), lr_, beta1_, beta2_, eps_,
                        wd_, count_, kv.first, hipBackendStream()) != FLHIP_OK)
      throw std::runtime_error(std::string("AdamOptimizer: ") + flhip_last_error());
  }
}

std::string AdamOptimizer::prettyString() const {
  std::ostringstream ss;                   // :81-89
  ss << "Adam";
  if (wd_ != 0) ss << " (weight decay=" << wd_ << ")";
  return ss.str();
}

std::string SGDOptimizer::prettyString() const {
  // SGDOptimizer.cpp:70-84
  std::ostringstream ss;
  ss << "SGD";
  if (wd_ != 0) ss << " (weight decay=" << wd_ << ")";
  if (useNesterov_ && mu_ != 0)
    ss << " (Nesterov momentum=" << mu_ << ")";
  else if (mu_ != 0)
    ss << " (momentum=" << mu_ << ")";
  return ss.str();
}

}  // namespace fl
