#include "Functions.h"

#include <algorithm>
#include <unordered_set>

#include "flhip.h"

namespace fl {

Variable::Variable(Tensor data, bool calcGrad)
    : data_(std::make_shared<Tensor>(std::move(data))), grad_(std::make_shared<SharedGrad>()) {
  grad_->calcGrad = calcGrad;
}

Variable::Variable(Tensor data, std::vector<Variable> inputs, GradFunc gradFunc)
    : data_(std::make_shared<Tensor>(std::move(data))), grad_(std::make_shared<SharedGrad>()) {
  // a result needs a gradient iff one of its inputs does (Variable.cpp:41-52)
  bool any = false;
  for (const auto& in : inputs) any = any || in.isCalcGrad();
  if (any) {
    grad_->calcGrad = true;
    grad_->inputs = std::move(inputs);
    grad_->gradFunc = std::move(gradFunc);
  }
}

Variable& Variable::grad() const {
  if (!grad_->calcGrad) throw std::logic_error("gradient calculation disabled for this Variable");
  if (!grad_->grad) throw std::logic_error("gradient not calculated yet for this Variable");
  return *grad_->grad;
}

void Variable::addGrad(const Variable& childGrad) {
  if (!grad_->calcGrad) return;
  // flashlight/fl/autograd/Variable.cpp:185-218
  if (childGrad.type() != type())
    throw std::invalid_argument("Variable::addGrad: gradient type does not match the variable");
  if (childGrad.shape() != shape())
    throw std::invalid_argument("Variable::addGrad: gradient shape does not match the variable");
  if (!grad_->grad) {
    grad_->grad.reset(new Variable(childGrad.tensor(), false));
    return;
  }
  Tensor sum(shape(), type());
  const int tag = type() == dtype::f32 ? FLHIP_F32 : FLHIP_BF16;
  if (type() != dtype::f32 && type() != dtype::bf16)
    throw std::runtime_error("Variable::addGrad: f32 and bf16 only");
  if (flhip_add(grad_->grad->tensor().device(), childGrad.tensor().device(), sum.device(),
                (size_t)sum.elements(), tag, hipBackendStream()) != FLHIP_OK)
    throw std::runtime_error(flhip_last_error());
  grad_->grad.reset(new Variable(sum, false));
}

std::vector<Variable> Variable::build() const {
  // depth-first post order = topological order (Variable.cpp:274-294)
  std::unordered_set<SharedGrad*> seen;
  std::vector<Variable> order;
  std::function<void(const Variable&)> visit = [&](const Variable& v) {
    if (seen.count(v.grad_.get())) return;
    for (const auto& in : v.grad_->inputs) visit(in);
    seen.insert(v.grad_.get());
    order.push_back(v);
  };
  visit(*this);
  return order;
}

void Variable::backward(const Variable& grad, bool retainGraph) {
  addGrad(grad);
  auto order = build();
  for (auto it = order.rbegin(); it != order.rend(); ++it) {
    Variable& v = *it;
    if (!v.grad_->gradFunc || !v.grad_->grad) continue;
    v.grad_->gradFunc(v.grad_->inputs, *v.grad_->grad);
    if (!retainGraph) v.grad_->inputs.clear();
  }
}

int derivePadding(int inSz, int filterSz, int stride, int pad, int dilation) {
  if (pad == static_cast<int>(PaddingMode::SAME)) {
    const int rem = inSz % stride;
    const int p = ((filterSz - 1) * dilation - (rem == 0 ? stride : rem) + 1 + 1) / 2;
    return std::max(p, 0);
  }
  return pad;
}

namespace {
// FL_VARIABLE_DTYPES_MATCH_CHECK (flashlight/fl/autograd/Functions.h:102-108)
void dtypesMatch(const char* fn, std::initializer_list<const Variable*> vars) {
  const Variable* first = nullptr;
  for (const Variable* v : vars) {
    if (v->isEmpty()) continue;
    if (!first) first = v;
    else if (v->type() != first->type())
      throw std::invalid_argument(std::string(fn) + " doesn't support binary operations with Variables of different types");
  }
}
// createAutogradPayload (flashlight/fl/autograd/Functions.h:84-89)
std::shared_ptr<detail::AutogradPayload> createPayload(std::initializer_list<const Variable*> vars) {
  for (const Variable* v : vars)
    if (v->isCalcGrad()) return std::make_shared<detail::AutogradPayload>();
  return nullptr;
}
AutogradExtension& ext(const Variable& v) { return getAutogradExtension(v.tensor().backendType()); }
}  // namespace

Variable conv2d(const Variable& input, const Variable& weights, int sx, int sy, int px, int py,
                int dx, int dy, int groups) {
  return conv2d(input, weights, Variable(), sx, sy, px, py, dx, dy, groups);
}

Variable conv2d(const Variable& input, const Variable& weights, const Variable& bias, int sx,
                int sy, int px, int py, int dx, int dy, int groups) {
  dtypesMatch("conv2d", {&input, &weights, &bias});
  const bool hasBias = bias.tensor().elements() > 0;
  auto payload = createPayload({&input, &weights, &bias});
  Tensor output = ext(input).conv2d(input.tensor(), weights.tensor(), bias.tensor(), sx, sy, px, py,
                                    dx, dy, groups, payload);

  auto gradFunc = [sx, sy, px, py, dx, dy, hasBias, groups, payload](
                      std::vector<Variable>& inputs, const Variable& gradOutput) {
    // Functions.cpp:1362-1452
    auto& in = inputs[0];
    auto& wt = inputs[1];
    AutogradExtension& e = ext(in);
    if (in.isCalcGrad()) {
      Tensor g = e.conv2dBackwardData(gradOutput.tensor(), in.tensor(), wt.tensor(), sx, sy, px, py,
                                      dx, dy, groups, nullptr, payload);
      in.addGrad(Variable(g, false));
    }
    const bool biasGrad = hasBias && inputs.size() > 2 && inputs[2].isCalcGrad();
    if (wt.isCalcGrad() || biasGrad) {
      // an empty bias tells the extension that no bias gradient is wanted (:1391-1395)
      const Tensor bs = biasGrad ? inputs[2].tensor() : Tensor();
      auto grads = e.conv2dBackwardFilterBias(gradOutput.tensor(), in.tensor(), wt.tensor(), bs, sx,
                                              sy, px, py, dx, dy, groups, nullptr, nullptr, payload);
      if (wt.isCalcGrad()) wt.addGrad(Variable(grads.first.astype(wt.type()), false));
      if (biasGrad) inputs[2].addGrad(Variable(grads.second.astype(inputs[2].type()), false));
    }
  };
  if (hasBias) return Variable(output, {input, weights, bias}, gradFunc);
  return Variable(output, {input, weights}, gradFunc);
}

Variable pool2d(const Variable& input, int wx, int wy, int sx, int sy, int px, int py,
                PoolingMode mode) {
  auto payload = createPayload({&input});
  Tensor output = ext(input).pool2d(input.tensor(), wx, wy, sx, sy, px, py, mode, payload);
  auto gradFunc = [wx, wy, sx, sy, px, py, mode, output, payload](std::vector<Variable>& inputs,
                                                                  const Variable& gradOutput) {
    // Functions.cpp:1472-1494
    auto& in = inputs[0];
    if (!in.isCalcGrad()) return;
    Tensor g = ext(in).pool2dBackward(gradOutput.tensor(), in.tensor(), output, wx, wy, sx, sy, px,
                                      py, mode, payload);
    in.addGrad(Variable(g, false));
  };
  return Variable(output, {input}, gradFunc);
}

Variable batchnorm(const Variable& input, const Variable& weight, const Variable& bias,
                   Variable& runningMean, Variable& runningVar, const std::vector<int>& axes,
                   bool train, double momentum, double epsilon) {
  dtypesMatch("batchnorm", {&input, &weight, &bias});
  auto payload = createPayload({&input, &weight, &bias});
  auto saveMean = std::make_shared<Tensor>();
  auto saveVar = std::make_shared<Tensor>();
  Tensor output = ext(input).batchnorm(*saveMean, *saveVar, input.tensor(), weight.tensor(),
                                       bias.tensor(), runningMean.tensor(), runningVar.tensor(), axes,
                                       train, momentum, epsilon, payload);
  auto gradFunc = [saveMean, saveVar, train, axes, epsilon, payload](std::vector<Variable>& inputs,
                                                                     const Variable& gradOutput) {
    // Functions.cpp:1526-1563
    auto& in = inputs[0];
    auto& wt = inputs[1];
    auto& bs = inputs[2];
    if (!in.isCalcGrad() && !wt.isCalcGrad() && !bs.isCalcGrad()) return;
    auto g = ext(in).batchnormBackward(gradOutput.tensor(), *saveMean, *saveVar, in.tensor(),
                                       wt.tensor(), axes, train, (float)epsilon, payload);
    in.addGrad(Variable(std::get<0>(g).astype(in.type()), false));
    if (!wt.isEmpty()) wt.addGrad(Variable(std::get<1>(g).reshaped(wt.shape()).astype(wt.type()), false));
    if (!bs.isEmpty()) bs.addGrad(Variable(std::get<2>(g).reshaped(bs.shape()).astype(bs.type()), false));
  };
  return Variable(output, {input, weight, bias}, gradFunc);
}

}  // namespace fl
