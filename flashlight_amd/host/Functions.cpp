#include "Functions.h"
#include "HipAutogradExtension.h"
#include "OpObserver.h"

#include <algorithm>
#include <tuple>
#include <unordered_map>
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
  detail::OpScope scope("addGrad");
  Tensor sum(shape(), type());
  if (type() != dtype::f32 && type() != dtype::bf16 && type() != dtype::f16)
    throw std::runtime_error("Variable::addGrad: f32, bf16 and f16 only");
  const int tag = type() == dtype::f32 ? FLHIP_F32 : type() == dtype::bf16 ? FLHIP_BF16 : FLHIP_F16;
  if (flhip_add(grad_->grad->tensor().device(), childGrad.tensor().device(), sum.device(),
                (size_t)sum.elements(), tag, hipBackendStream()) != FLHIP_OK)
    throw std::runtime_error(flhip_last_error());
  if (scope.on()) scope.done({grad_->grad->tensor(), childGrad.tensor()}, {sum});
  grad_->grad.reset(new Variable(sum, false));
}

void Variable::setCalcGrad(bool calcGrad) {
  grad_->calcGrad = calcGrad;
  if (!calcGrad) {
    grad_->gradFunc = nullptr;
    grad_->inputs.clear();
    grad_->grad.reset();
  }
}

namespace {
struct ParamCasts {
  dtype to;
  std::unordered_map<const void*, Variable> nodes;
};
ParamCasts* g_paramCasts = nullptr;
}  // namespace

detail::ParamCastScope::ParamCastScope(const std::vector<Variable>& params, dtype to) {
  if (g_paramCasts) return;   // an outer scope made the casts
  std::vector<Variable> todo;
  std::vector<Tensor> src;
  std::unordered_set<const void*> seen;
  for (const auto& p : params)
    if (!p.isEmpty() && p.type() != to && seen.insert(p.id()).second) {
      todo.push_back(p);
      src.push_back(p.tensor());
    }
  if (todo.empty()) return;
  const std::vector<Tensor> converted = Tensor::astypeMany(src, to);
  auto* casts = new ParamCasts{to, {}};
  for (size_t i = 0; i < todo.size(); ++i) casts->nodes.emplace(todo[i].id(), todo[i].castNode(converted[i]));
  g_paramCasts = casts;
  owner_ = true;
}

detail::ParamCastScope::~ParamCastScope() {
  if (!owner_) return;
  delete g_paramCasts;
  g_paramCasts = nullptr;
}

Variable Variable::castNode(const Tensor& converted) const {
  const dtype oldType = type();
  auto gradFunc = [oldType](std::vector<Variable>& inputs, const Variable& gradOutput) {
    inputs[0].addGrad(Variable(gradOutput.tensor().astype(oldType), false));
  };
  Variable out(converted, {*this}, gradFunc);
  out.grad_->isCast = out.grad_->calcGrad;
  return out;
}

Variable Variable::astype(dtype newType) const {
  if (newType == type()) return *this;
  if (g_paramCasts && g_paramCasts->to == newType) {
    const auto it = g_paramCasts->nodes.find(id());
    if (it != g_paramCasts->nodes.end()) return it->second;
  }
  return castNode(tensor().astype(newType));
}

void Variable::addGradWide(const Tensor& grad) {
  if (!grad_->calcGrad) return;
  if (grad_->isCast && !grad_->inputs.empty() && grad.type() != type() && grad_->inputs[0].type() == grad.type()) {
    grad_->inputs[0].addGrad(Variable(grad, false));
    return;
  }
  addGrad(Variable(grad.astype(type()), false));
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
                int dx, int dy, int groups, std::shared_ptr<detail::ConvBenchmarks> benchmarks) {
  return conv2d(input, weights, Variable(), sx, sy, px, py, dx, dy, groups, std::move(benchmarks));
}

Variable conv2d(const Variable& input, const Variable& weights, const Variable& bias, int sx,
                int sy, int px, int py, int dx, int dy, int groups,
                std::shared_ptr<detail::ConvBenchmarks> benchmarks) {
  dtypesMatch("conv2d", {&input, &weights, &bias});
  const bool hasBias = bias.tensor().elements() > 0;
  auto payload = createPayload({&input, &weights, &bias});
  Tensor output = ext(input).conv2d(input.tensor(), weights.tensor(), bias.tensor(), sx, sy, px, py,
                                    dx, dy, groups, payload);

  auto gradFunc = [sx, sy, px, py, dx, dy, hasBias, groups, benchmarks, payload](
                      std::vector<Variable>& inputs, const Variable& gradOutput) {
    // Functions.cpp:1362-1452
    auto& in = inputs[0];
    auto& wt = inputs[1];
    AutogradExtension& e = ext(in);
    // The benchmarks of the two passes: made on the first backward pass in benchmark mode (:1372-1388) and handed
    // to the extension on every pass from then on (the reference hands them over only on the pass that makes
    // them), so that the choice they arrive at is used once the timings are complete, also with the mode off again.
    std::shared_ptr<DynamicBenchmark> dataBench, filterBench, biasBench;
    if (benchmarks) {
      if (DynamicBenchmark::getBenchmarkMode()) {
        if (!benchmarks->bwdFilterBenchmark) benchmarks->bwdFilterBenchmark = e.createBenchmarkOptions();
        if (!benchmarks->bwdDataBenchmark) benchmarks->bwdDataBenchmark = e.createBenchmarkOptions();
        if (!benchmarks->bwdBiasBenchmark) benchmarks->bwdBiasBenchmark = e.createBenchmarkOptions();
      }
      dataBench = benchmarks->bwdDataBenchmark;
      filterBench = benchmarks->bwdFilterBenchmark;
      biasBench = benchmarks->bwdBiasBenchmark;
    }
    if (in.isCalcGrad()) {
      auto* hip = detail::fusedGradAdd() ? dynamic_cast<HipAutogradExtension*>(&e) : nullptr;
      if (hip && in.isGradAvailable() && in.grad().type() == gradOutput.type() && in.grad().shape() == in.shape()) {
        // the second gradient of this variable (the first came down the shortcut): summed where
        // the pass writes its result
        in.replaceGrad(hip->conv2dBackwardDataAdd(gradOutput.tensor(), in.tensor(), wt.tensor(), in.grad().tensor(),
                                                  sx, sy, px, py, dx, dy, groups));
      } else {
        Tensor g = e.conv2dBackwardData(gradOutput.tensor(), in.tensor(), wt.tensor(), sx, sy, px, py,
                                        dx, dy, groups, dataBench, payload);
        in.addGrad(Variable(g, false));
      }
    }
    const bool biasGrad = hasBias && inputs.size() > 2 && inputs[2].isCalcGrad();
    if (wt.isCalcGrad() || biasGrad) {
      // an empty bias tells the extension that no bias gradient is wanted (:1391-1395)
      const Tensor bs = biasGrad ? inputs[2].tensor() : Tensor();
      auto grads = e.conv2dBackwardFilterBias(gradOutput.tensor(), in.tensor(), wt.tensor(), bs, sx,
                                              sy, px, py, dx, dy, groups, filterBench, biasBench, payload);
      if (wt.isCalcGrad()) wt.addGradWide(grads.first);
      if (biasGrad) inputs[2].addGradWide(grads.second);
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
  // the BatchNorm and LayerNorm modules keep f32 parameters for 16-bit inputs
  // (flashlight/fl/nn/modules/BatchNorm.cpp:86-88), so f32 is accepted beside the input type
  for (const Variable* v : {&weight, &bias})
    if (!v->isEmpty() && v->type() != input.type() && v->type() != dtype::f32)
      throw std::invalid_argument("batchnorm: parameters must have the input's type or f32");
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

namespace {
bool g_fusedGradAdd = true;
}
void detail::setFusedGradAdd(bool on) { g_fusedGradAdd = on; }
bool detail::fusedGradAdd() { return g_fusedGradAdd; }

Variable detail::batchnormRelu(const Variable& input, const Variable& weight, const Variable& bias,
                               Variable& runningMean, Variable& runningVar, const std::vector<int>& axes,
                               double momentum, double epsilon, const Variable& residual) {
  auto* hip = dynamic_cast<HipAutogradExtension*>(&ext(input));
  const bool perActivation = !axes.empty() && *std::min_element(axes.begin(), axes.end()) == 0;
  if (!hip || perActivation) {
    Variable y = batchnorm(input, weight, bias, runningMean, runningVar, axes, true, momentum, epsilon);
    return relu(residual.isEmpty() ? y : y + residual);
  }
  for (const Variable* v : {&weight, &bias})
    if (!v->isEmpty() && v->type() != input.type() && v->type() != dtype::f32)
      throw std::invalid_argument("batchnormRelu: parameters must have the input's type or f32");
  const bool hasResidual = !residual.isEmpty();
  if (hasResidual) dtypesMatch("batchnormRelu", {&input, &residual});
  auto payload = createPayload({&input, &weight, &bias, &residual});
  auto saveMean = std::make_shared<Tensor>();
  auto saveVar = std::make_shared<Tensor>();
  Tensor output = hip->batchnormRelu(*saveMean, *saveVar, input.tensor(), weight.tensor(), bias.tensor(),
                                     runningMean.tensor(), runningVar.tensor(), axes, momentum, epsilon,
                                     residual.tensor(), payload);
  auto gradFunc = [saveMean, saveVar, axes, output, hasResidual, payload](std::vector<Variable>& inputs,
                                                                          const Variable& gradOutput) {
    auto& in = inputs[0];
    auto& wt = inputs[1];
    auto& bs = inputs[2];
    const bool resGrad = hasResidual && inputs[3].isCalcGrad();
    if (!in.isCalcGrad() && !wt.isCalcGrad() && !bs.isCalcGrad() && !resGrad) return;
    auto* h = dynamic_cast<HipAutogradExtension*>(&ext(in));
    auto g = h->batchnormReluBackward(gradOutput.tensor(), output, *saveMean, *saveVar, in.tensor(), wt.tensor(),
                                      axes, resGrad, payload);
    in.addGrad(Variable(std::get<0>(g).astype(in.type()), false));
    if (!wt.isEmpty()) wt.addGrad(Variable(std::get<1>(g).reshaped(wt.shape()).astype(wt.type()), false));
    if (!bs.isEmpty()) bs.addGrad(Variable(std::get<2>(g).reshaped(bs.shape()).astype(bs.type()), false));
    if (resGrad) inputs[3].addGrad(Variable(std::get<3>(g), false));
  };
  if (hasResidual) return Variable(output, {input, weight, bias, residual}, gradFunc);
  return Variable(output, {input, weight, bias}, gradFunc);
}

std::tuple<Variable, Variable, Variable> rnn(const Variable& input, const Variable& hiddenState,
                                             const Variable& cellState, const Variable& weights,
                                             int hiddenSize, int numLayers, RnnMode mode,
                                             bool bidirectional, float dropProb) {
  auto payload = createPayload({&input, &hiddenState, &cellState, &weights});
  Tensor output, hiddenOut, cellOut;
  std::tie(output, hiddenOut, cellOut) =
      ext(input).rnn(input.tensor(), hiddenState.tensor(), cellState.tensor(), weights.tensor(), hiddenSize,
                     numLayers, mode, bidirectional, dropProb, payload);
  auto gradData = std::make_shared<detail::RNNGradData>();
  auto gradFunc = [output, numLayers, hiddenSize, mode, bidirectional, dropProb, gradData, payload](
                      std::vector<Variable>& inputs, const Variable&) {
    auto& in = inputs[0];
    auto& hs = inputs[1];
    auto& cs = inputs[2];
    auto& wt = inputs[3];
    if (!(in.isCalcGrad() || hs.isCalcGrad() || cs.isCalcGrad() || wt.isCalcGrad())) return;
    auto g = ext(in).rnnBackward(in.tensor(), hs.tensor(), cs.tensor(), wt.tensor(), gradData, output, numLayers,
                                 hiddenSize, mode, bidirectional, dropProb, payload);
    in.addGrad(Variable(std::get<0>(g).astype(in.type()), false));
    if (!hs.isEmpty()) hs.addGrad(Variable(std::get<1>(g).astype(hs.type()), false));
    if (!cs.isEmpty()) cs.addGrad(Variable(std::get<2>(g).astype(cs.type()), false));
    wt.addGrad(Variable(std::get<3>(g).astype(wt.type()), false));
  };
  // one node that owns the backward call; the three outputs hang off it and only record
  // their gradients (Functions.cpp:1675-1703)
  Variable dummy(Tensor(), {input, hiddenState, cellState, weights}, gradFunc);
  auto record = [gradData](Tensor detail::RNNGradData::*slot) {
    return [gradData, slot](std::vector<Variable>& inputs, const Variable& gradOutput) {
      if (!inputs[0].isGradAvailable()) inputs[0].addGrad(Variable(Tensor(), false));
      (*gradData).*slot = gradOutput.tensor();
    };
  };
  Variable yv(output, {dummy}, record(&detail::RNNGradData::dy));
  Variable hyv(hiddenOut, {dummy}, record(&detail::RNNGradData::dhy));
  Variable cyv(cellOut, {dummy}, record(&detail::RNNGradData::dcy));
  return std::make_tuple(yv, hyv, cyv);
}

namespace {
int tagOf(dtype t, const char* fn) {
  if (t == dtype::f32) return FLHIP_F32;
  if (t == dtype::bf16) return FLHIP_BF16;
  if (t == dtype::f16) return FLHIP_F16;
  throw std::runtime_error(std::string(fn) + ": f32, bf16 and f16 only");
}
void check(int rc) {
  if (rc == FLHIP_INVALID_ARGUMENT) throw std::invalid_argument(flhip_last_error());
  if (rc != FLHIP_OK) throw std::runtime_error(flhip_last_error());
}
}  // namespace

Variable add(const Variable& lhs, const Variable& rhs) {
  dtypesMatch("add", {&lhs, &rhs});
  if (lhs.shape() != rhs.shape())
    throw std::invalid_argument("add: shapes must match (no broadcasting on this backend)");
  detail::OpScope scope("add");
  const int tag = tagOf(lhs.type(), "add");
  Tensor out(lhs.shape(), lhs.type());
  check(flhip_add(lhs.tensor().device(), rhs.tensor().device(), out.device(), (size_t)out.elements(), tag,
                  hipBackendStream()));
  if (scope.on()) scope.done({lhs.tensor(), rhs.tensor()}, {out});
  auto gradFunc = [](std::vector<Variable>& inputs, const Variable& gradOutput) {
    inputs[0].addGrad(Variable(gradOutput.tensor(), false));
    inputs[1].addGrad(Variable(gradOutput.tensor(), false));
  };
  return Variable(out, {lhs, rhs}, gradFunc);
}

Variable detail::affine(const Variable& input, const Variable& weight, const Variable& bias, Dim outer,
                        Dim mid, Dim inner, bool scalar) {
  dtypesMatch("affine", {&input, &weight, &bias});
  if (outer * mid * inner != input.elements() || weight.elements() != (scalar ? 1 : mid) ||
      bias.elements() != weight.elements())
    throw std::invalid_argument("affine: the view or the parameters do not match the input");
  const int tag = tagOf(input.type(), "affine");
  Tensor out(input.shape(), input.type());
  check(flhip_affine_fwd(input.tensor().device(), weight.tensor().device(), bias.tensor().device(),
                         out.device(), outer, mid, inner, scalar ? 1 : 0, tag, hipBackendStream()));
  auto gradFunc = [outer, mid, inner, scalar, tag](std::vector<Variable>& inputs,
                                                   const Variable& gradOutput) {
    auto& x = inputs[0];
    auto& w = inputs[1];
    auto& b = inputs[2];
    const bool sums = w.isCalcGrad() || b.isCalcGrad();
    Tensor dx = x.isCalcGrad() ? Tensor(x.shape(), x.type()) : Tensor();
    Tensor dw = sums ? Tensor(w.shape(), dtype::f32) : Tensor();
    Tensor db = sums ? Tensor(b.shape(), dtype::f32) : Tensor();
    const size_t wsBytes = sums ? flhip_affine_bwd_workspace_bytes(outer, mid, inner, scalar ? 1 : 0) : 0;
    Tensor ws = wsBytes ? Tensor({(Dim)wsBytes}, dtype::u8) : Tensor();
    check(flhip_affine_bwd(gradOutput.tensor().device(), x.tensor().device(), w.tensor().device(),
                           dx.device(), static_cast<float*>(dw.device()),
                           static_cast<float*>(db.device()), outer, mid, inner, scalar ? 1 : 0, tag,
                           ws.device(), wsBytes, hipBackendStream()));
    if (x.isCalcGrad()) x.addGrad(Variable(dx, false));
    if (w.isCalcGrad()) w.addGrad(Variable(dw.astype(w.type()), false));
    if (b.isCalcGrad()) b.addGrad(Variable(db.astype(b.type()), false));
  };
  return Variable(out, {input, weight, bias}, gradFunc);
}

Variable embedding(const Variable& input, const Variable& embeddings) {
  if (input.ndim() >= 4) throw std::invalid_argument("embedding input must have 3 or fewer dims");   // as the reference
  if (input.type() != dtype::s32) throw std::invalid_argument("embedding: indices must be s32 on this backend");
  if (embeddings.ndim() != 2 || input.elements() == 0) throw std::invalid_argument("embedding: a [dim, tokens] table and at least one index");
  detail::OpScope scope("embedding");
  const int tag = tagOf(embeddings.type(), "embedding");
  const Dim dim = embeddings.dim(0), tokens = embeddings.dim(1), n = input.elements();
  std::vector<Dim> rDims{dim};
  for (int i = 0; i < input.ndim(); ++i) rDims.push_back(input.dim(i));
  Tensor out{Shape(rDims), embeddings.type()};
  check(flhip_embedding_fwd(static_cast<const int32_t*>(input.tensor().device()), embeddings.tensor().device(), out.device(),
                            (int64_t)n, (int32_t)dim, (int32_t)tokens, tag, hipBackendStream()));
  if (scope.on()) scope.done({input.tensor(), embeddings.tensor()}, {out});
  auto gradFunc = [n, dim, tokens, tag](std::vector<Variable>& inputs, const Variable& gradOutput) {
    auto& w = inputs[1];
    if (!w.isCalcGrad()) return;
    detail::OpScope scope("embeddingBackward");
    Tensor dw(w.shape(), w.type());
    check(flhip_embedding_bwd(static_cast<const int32_t*>(inputs[0].tensor().device()), gradOutput.tensor().device(),
                              dw.device(), (int64_t)n, (int32_t)dim, (int32_t)tokens, tag, hipBackendStream()));
    if (scope.on()) scope.done({gradOutput.tensor(), inputs[0].tensor()}, {dw});
    w.addGrad(Variable(dw, false));
  };
  return Variable(out, {input, embeddings}, gradFunc);
}

Variable prelu(const Variable& input, const Variable& weight) {
  dtypesMatch("prelu", {&input, &weight});
  if (input.ndim() < 1 || input.elements() == 0) throw std::invalid_argument("prelu: empty input");
  const Dim d0 = input.dim(0), outer = input.elements() / d0;
  const bool scalar = weight.elements() == 1;
  // tileAs (Functions.cpp: tileAs) repeats the parameter along dimension 0; one element or a full set are the cases built
  if (!scalar && weight.elements() != d0)
    throw std::invalid_argument("prelu: the parameter has one element, or one per index of the input's first dimension");
  detail::OpScope scope("prelu");
  const int tag = tagOf(input.type(), "prelu");
  Tensor out(input.shape(), input.type());
  check(flhip_prelu_fwd(input.tensor().device(), weight.tensor().device(), out.device(), outer, d0, scalar ? 1 : 0, tag,
                        hipBackendStream()));
  if (scope.on()) scope.done({input.tensor(), weight.tensor()}, {out});
  auto gradFunc = [outer, d0, scalar, tag](std::vector<Variable>& inputs, const Variable& gradOutput) {
    auto& x = inputs[0];
    auto& w = inputs[1];
    if (!x.isCalcGrad() && !w.isCalcGrad()) return;
    detail::OpScope scope("preluBackward");
    Tensor dx = x.isCalcGrad() ? Tensor(x.shape(), x.type()) : Tensor();
    Tensor dw = w.isCalcGrad() ? Tensor(w.shape(), dtype::f32) : Tensor();
    const size_t wsBytes = w.isCalcGrad() ? flhip_prelu_bwd_workspace_bytes(outer, d0, scalar ? 1 : 0) : 0;
    Tensor ws = wsBytes ? Tensor({(Dim)wsBytes}, dtype::u8) : Tensor();
    check(flhip_prelu_bwd(gradOutput.tensor().device(), x.tensor().device(), w.tensor().device(), dx.device(),
                          static_cast<float*>(dw.device()), outer, d0, scalar ? 1 : 0, tag, ws.device(), wsBytes,
                          hipBackendStream()));
    if (scope.on()) scope.done({gradOutput.tensor(), x.tensor()}, {dx});
    if (x.isCalcGrad()) x.addGrad(Variable(dx, false));
    if (w.isCalcGrad()) w.addGrad(Variable(dw.astype(w.type()), false));
  };
  return Variable(out, {input, weight}, gradFunc);
}

Variable relu(const Variable& input) {
  detail::OpScope scope("relu");
  Tensor out(input.shape(), input.type());
  check(flhip_relu_fwd(input.tensor().device(), out.device(), (size_t)out.elements(),
                       tagOf(input.type(), "relu"), hipBackendStream()));
  if (scope.on()) scope.done({input.tensor()}, {out});
  auto gradFunc = [](std::vector<Variable>& inputs, const Variable& gradOutput) {
    // mask = (input > 0) (Functions.cpp:333-335)
    auto& in = inputs[0];
    if (!in.isCalcGrad()) return;
    detail::OpScope scope("reluBackward");
    Tensor g(in.shape(), gradOutput.type());
    check(flhip_relu_bwd(gradOutput.tensor().device(), in.tensor().device(), g.device(),
                         (size_t)g.elements(), tagOf(g.type(), "relu"), hipBackendStream()));
    if (scope.on()) scope.done({gradOutput.tensor(), in.tensor()}, {g});
    in.addGrad(Variable(g, false));
  };
  return Variable(out, {input}, gradFunc);
}

namespace {
// y = f(x) / dx = dy f'(x) through flhip_act_fwd / _bwd; the closure keeps the input (the reference's closures keep
// the result for tanh, clamp and sigmoid: the same function of the same input)
Variable activation(const char* name, int op, const Variable& input, double a, double b) {
  detail::OpScope scope(name);
  Tensor out(input.shape(), input.type());
  check(flhip_act_fwd(op, input.tensor().device(), out.device(), (size_t)out.elements(), a, b,
                      tagOf(input.type(), name), hipBackendStream()));
  if (scope.on()) scope.done({input.tensor()}, {out});
  auto gradFunc = [op, a, b, name](std::vector<Variable>& inputs, const Variable& gradOutput) {
    auto& in = inputs[0];
    if (!in.isCalcGrad()) return;
    detail::OpScope scope("activationBackward");
    Tensor g(in.shape(), gradOutput.type());
    check(flhip_act_bwd(op, gradOutput.tensor().device(), in.tensor().device(), g.device(), (size_t)g.elements(), a, b,
                        tagOf(g.type(), name), hipBackendStream()));
    if (scope.on()) scope.done({gradOutput.tensor(), in.tensor()}, {g});
    in.addGrad(Variable(g, false));
  };
  return Variable(out, {input}, gradFunc);
}
}  // namespace

Variable elu(const Variable& input, double alpha) { return activation("elu", FLHIP_ACT_ELU, input, alpha, 0.0); }
Variable clamp(const Variable& input, double lo, double hi) {
  if (lo > hi) throw std::invalid_argument("clamp: lo must not exceed hi");
  return activation("clamp", FLHIP_ACT_CLAMP, input, lo, hi);
}
Variable tanh(const Variable& input) { return activation("tanh", FLHIP_ACT_TANH, input, 0.0, 0.0); }
Variable log(const Variable& input) { return activation("log", FLHIP_ACT_LOG, input, 0.0, 0.0); }
Variable sigmoid(const Variable& input) { return activation("sigmoid", FLHIP_ACT_SIGMOID, input, 0.0, 0.0); }
Variable swish(const Variable& input, double beta) { return activation("swish", FLHIP_ACT_SWISH, input, beta, 0.0); }
Variable scale(const Variable& input, double factor) { return activation("scale", FLHIP_ACT_SCALE, input, factor, 0.0); }
Variable leakyRelu(const Variable& input, double slope) { return activation("leakyRelu", FLHIP_ACT_LEAKY, input, slope, 0.0); }
Variable thresholdRelu(const Variable& input, double threshold) {
  return activation("thresholdRelu", FLHIP_ACT_THRESHOLD, input, threshold, 0.0);
}

Variable gatedlinearunit(const Variable& input, int dim) {
  // Functions.cpp:1567-1579
  if (dim < 0 || dim >= input.ndim())
    throw std::invalid_argument("gatedlinearunit - passed dim is great than the number of dimensions of the input.");
  const Shape& in = input.shape();
  if (in.dim(dim) % 2 == 1) throw std::invalid_argument("halving dimension must be even for GLU");
  // column-major: the dimensions before `dim` are the fast ones
  long long m = in.dim(dim) / 2, outer = 1;
  for (int i = 0; i < dim; ++i) m *= in.dim(i);
  for (int i = dim + 1; i < in.ndim(); ++i) outer *= in.dim(i);
  std::vector<Dim> od = in.get();
  od[(size_t)dim] /= 2;
  detail::OpScope scope("gatedlinearunit");
  Tensor out{Shape(od), input.type()};
  if (out.elements() > 0)
    check(flhip_glu_fwd(input.tensor().device(), out.device(), outer, m, tagOf(input.type(), "gatedlinearunit"),
                        hipBackendStream()));
  if (scope.on()) scope.done({input.tensor()}, {out});
  auto gradFunc = [outer, m](std::vector<Variable>& inputs, const Variable& gradOutput) {
    auto& in = inputs[0];
    if (!in.isCalcGrad()) return;
    detail::OpScope scope("gatedlinearunitBackward");
    Tensor g(in.shape(), gradOutput.type());
    if (g.elements() > 0)
      check(flhip_glu_bwd(gradOutput.tensor().device(), in.tensor().device(), g.device(), outer, m,
                          tagOf(g.type(), "gatedlinearunit"), hipBackendStream()));
    if (scope.on()) scope.done({gradOutput.tensor(), in.tensor()}, {g});
    in.addGrad(Variable(g, false));
  };
  return Variable(out, {input}, gradFunc);
}

unsigned long long nextSeed();   // Modules.cpp: the process-wide generator

Variable dropout(const Variable& input, double p) {
  if (!(p > 0.0)) return input;                                   // Functions.cpp:1778, 1782-1784
  if (p >= 1.0) throw std::invalid_argument("dropout: the probability must be below 1");
  const unsigned long long seed = nextSeed();
  const uint32_t lo = (uint32_t)seed, hi = (uint32_t)(seed >> 32);
  detail::OpScope scope("dropout");
  Tensor out(input.shape(), input.type());
  check(flhip_dropout(input.tensor().device(), out.device(), (size_t)out.elements(), p, lo, hi,
                      tagOf(input.type(), "dropout"), hipBackendStream()));
  if (scope.on()) scope.done({input.tensor()}, {out});
  auto gradFunc = [p, lo, hi](std::vector<Variable>& inputs, const Variable& gradOutput) {
    auto& in = inputs[0];
    if (!in.isCalcGrad()) return;
    detail::OpScope scope("dropoutBackward");
    Tensor g(in.shape(), gradOutput.type());
    check(flhip_dropout(gradOutput.tensor().device(), g.device(), (size_t)g.elements(), p, lo, hi,
                        tagOf(g.type(), "dropout"), hipBackendStream()));
    if (scope.on()) scope.done({gradOutput.tensor()}, {g});
    in.addGrad(Variable(g, false));
  };
  return Variable(out, {input}, gradFunc);
}

namespace {
// rows x cols view of a weight for WeightNorm: the kept dimension first (fastest) or last
void weightNormView(const Shape& s, int dim, long long* rows, long long* cols, int* rowsFast) {
  const int nd = s.ndim();
  if (!(nd >= 1 && (dim == 0 || dim == nd - 1)))
    throw std::invalid_argument("Wrong dimension for Weight Norm: " + std::to_string(dim));   // WeightNorm.cpp:62-64
  *rows = s.dim(dim);
  *cols = s.elements() / std::max<long long>(1, s.dim(dim));
  // a one-dimensional or single-row weight: either view is the same memory
  *rowsFast = (dim == 0 && nd > 1) ? 1 : 0;
  if (*rows <= 0 || *cols <= 0) throw std::invalid_argument("WeightNorm: empty weight");
}
}  // namespace

Tensor rowNorm(const Tensor& v, int dim) {
  long long rows, cols;
  int fast;
  weightNormView(v.shape(), dim, &rows, &cols, &fast);
  std::vector<Dim> gd((size_t)v.ndim(), 1);
  gd[(size_t)dim] = rows;
  Tensor n{Shape(gd), v.type()};
  check(flhip_rownorm(v.device(), n.device(), rows, cols, fast, tagOf(v.type(), "weightNorm"), hipBackendStream()));
  return n;
}

Variable weightNorm(const Variable& v, const Variable& g, int dim) {
  dtypesMatch("weightNorm", {&v, &g});
  long long rows, cols;
  int fast;
  weightNormView(v.shape(), dim, &rows, &cols, &fast);
  if (g.tensor().elements() != rows) throw std::invalid_argument("weightNorm: g must have one element per index of dim");
  const int tag = tagOf(v.type(), "weightNorm");
  detail::OpScope scope("weightNorm");
  Tensor w(v.shape(), v.type());
  check(flhip_weightnorm_fwd(v.tensor().device(), g.tensor().device(), w.device(), rows, cols, fast, tag, hipBackendStream()));
  if (scope.on()) scope.done({v.tensor(), g.tensor()}, {w});
  auto gradFunc = [rows, cols, fast, tag](std::vector<Variable>& inputs, const Variable& gradOutput) {
    auto& vv = inputs[0];
    auto& gg = inputs[1];
    if (!vv.isCalcGrad() && !gg.isCalcGrad()) return;
    detail::OpScope scope("weightNormBackward");
    Tensor dv(vv.shape(), vv.type()), dg(gg.shape(), gg.type());
    const Tensor go = gradOutput.tensor().type() == vv.type() ? gradOutput.tensor() : gradOutput.tensor().astype(vv.type());
    check(flhip_weightnorm_bwd(go.device(), vv.tensor().device(), gg.tensor().device(), dv.device(), dg.device(), rows,
                               cols, fast, tag, hipBackendStream()));
    if (scope.on()) scope.done({go, vv.tensor(), gg.tensor()}, {dv, dg});
    if (vv.isCalcGrad()) vv.addGrad(Variable(dv, false));
    if (gg.isCalcGrad()) gg.addGrad(Variable(dg, false));
  };
  return Variable(w, {v, g}, gradFunc);
}

Variable padding(const Variable& input, const std::vector<std::pair<int, int>>& pad, double val) {
  const int nd = input.ndim();
  if ((int)pad.size() > nd)
    throw std::invalid_argument("padding: number of padding dimensions exceeds number of input dimensions");
  if (nd > 4) throw std::invalid_argument("padding: at most four dimensions");
  int64_t dims[4] = {1, 1, 1, 1};
  int32_t before[4] = {0, 0, 0, 0}, after[4] = {0, 0, 0, 0};
  std::vector<Dim> od = input.shape().get();
  for (int i = 0; i < nd; ++i) dims[i] = input.shape().dim(i);
  for (size_t i = 0; i < pad.size(); ++i) {
    if (pad[i].first < 0 || pad[i].second < 0) throw std::invalid_argument("padding: widths must not be negative");
    before[i] = pad[i].first;
    after[i] = pad[i].second;
    od[i] += pad[i].first + pad[i].second;
  }
  const int tag = tagOf(input.type(), "padding");
  detail::OpScope scope("padding");
  Tensor out{Shape(od), input.type()};
  if (input.tensor().elements() > 0)
    check(flhip_pad_fwd(input.tensor().device(), out.device(), dims, before, after, val, tag, hipBackendStream()));
  if (scope.on()) scope.done({input.tensor()}, {out});
  std::vector<int64_t> dv(dims, dims + 4);
  std::vector<int32_t> bv(before, before + 4), av(after, after + 4);
  auto gradFunc = [dv, bv, av, tag](std::vector<Variable>& inputs, const Variable& gradOutput) {
    auto& in = inputs[0];
    if (!in.isCalcGrad()) return;
    detail::OpScope scope("paddingBackward");
    Tensor g(in.shape(), gradOutput.type());
    if (g.elements() > 0)
      check(flhip_pad_bwd(gradOutput.tensor().device(), g.device(), dv.data(), bv.data(), av.data(),
                          tagOf(g.type(), "padding"), hipBackendStream()));
    if (scope.on()) scope.done({gradOutput.tensor()}, {g});
    in.addGrad(Variable(g, false));
  };
  return Variable(out, {input}, gradFunc);
}

Variable narrow(const Variable& input, int dim, long long start, long long size) {
  const int nd = input.ndim();
  if (dim < 0 || dim >= nd || nd > 4) throw std::invalid_argument("narrow: dimension out of range");
  const long long ext = input.shape().dim(dim);
  if (start < 0 || size <= 0 || start + size > ext) throw std::invalid_argument("narrow: range outside the dimension");
  // the slice as the inner box of the input: the kernels of fl::padding with the roles exchanged
  std::vector<int64_t> dims(4, 1);
  std::vector<int32_t> before(4, 0), after(4, 0);
  std::vector<Dim> od = input.shape().get();
  for (int i = 0; i < nd; ++i) dims[(size_t)i] = input.shape().dim(i);
  dims[(size_t)dim] = size;
  before[(size_t)dim] = (int32_t)start;
  after[(size_t)dim] = (int32_t)(ext - start - size);
  od[(size_t)dim] = size;
  detail::OpScope scope("narrow");
  Tensor out{Shape(od), input.type()};
  check(flhip_pad_bwd(input.tensor().device(), out.device(), dims.data(), before.data(), after.data(),
                      tagOf(input.type(), "narrow"), hipBackendStream()));
  if (scope.on()) scope.done({input.tensor()}, {out});
  auto gradFunc = [dims, before, after](std::vector<Variable>& inputs, const Variable& gradOutput) {
    auto& in = inputs[0];
    if (!in.isCalcGrad()) return;
    detail::OpScope scope("narrowBackward");
    Tensor g(in.shape(), gradOutput.type());
    check(flhip_pad_fwd(gradOutput.tensor().device(), g.device(), dims.data(), before.data(), after.data(), 0.0,
                        tagOf(g.type(), "narrow"), hipBackendStream()));
    if (scope.on()) scope.done({gradOutput.tensor()}, {g});
    in.addGrad(Variable(g, false));
  };
  return Variable(out, {input}, gradFunc);
}

Variable moddims(const Variable& input, const Shape& dims) {
  // a 0 keeps the input's dimension, one -1 is inferred from the element count
  // (Functions.cpp:969-1008)
  std::vector<Dim> d = dims.get();
  for (size_t i = 0; i < d.size(); ++i)
    if (d[i] == 0) {
      if ((int)i >= input.tensor().ndim())
        throw std::invalid_argument("moddims: tried to infer dimension " + std::to_string(i) +
                                    " which exceeds the number of dimensions of the input.");
      d[i] = input.tensor().dim((int)i);
    }
  Dim known = 1;
  int infer = -1;
  for (size_t i = 0; i < d.size(); ++i) {
    if (d[i] == -1) {
      if (infer >= 0) throw std::invalid_argument("moddims: too many dimensions infer");
      infer = (int)i;
    } else {
      known *= d[i];
    }
  }
  if (infer >= 0) d[infer] = known ? input.tensor().elements() / known : 0;
  const Shape target(d);
  if (target.elements() != input.tensor().elements())
    throw std::invalid_argument("moddims: mismatched number of elements");
  const Shape inShape = input.shape();
  auto gradFunc = [inShape](std::vector<Variable>& inputs, const Variable& gradOutput) {
    inputs[0].addGrad(Variable(gradOutput.tensor().reshaped(inShape), false));
  };
  return Variable(input.tensor().reshaped(target), {input}, gradFunc);
}

namespace {
Tensor reorderTensor(const Tensor& in, const std::vector<int>& perm) {
  detail::OpScope scope("reorder");
  int64_t dims[4] = {1, 1, 1, 1};
  int32_t pm[4] = {0, 1, 2, 3};
  for (int i = 0; i < in.ndim(); ++i) dims[i] = in.dim(i);
  for (size_t i = 0; i < perm.size(); ++i) pm[i] = perm[i];
  std::vector<Dim> oshape(in.ndim());
  for (int i = 0; i < in.ndim(); ++i) oshape[i] = in.dim(perm[i]);
  Tensor out(Shape(oshape), in.type());
  check(flhip_reorder(in.device(), out.device(), dims, pm, tagOf(in.type(), "reorder"), hipBackendStream()));
  if (scope.on()) scope.done({in}, {out}, {pm[0], pm[1], pm[2], pm[3]});
  return out;
}
}  // namespace

Variable reorder(const Variable& input, const Shape& dims) {
  const int nd = input.ndim();
  if (dims.ndim() != nd || nd > 4)
    throw std::invalid_argument("reorder: expects one entry per dimension of the input (at most 4)");
  std::vector<int> perm(nd), inverse(nd);
  std::vector<bool> seen(nd, false);
  for (int i = 0; i < nd; ++i) {
    const Dim d = dims.dim(i);
    if (d < 0 || d >= nd || seen[(size_t)d]) throw std::invalid_argument("reorder: not a permutation of the dimensions");
    seen[(size_t)d] = true;
    perm[i] = (int)d;
    inverse[(size_t)d] = i;
  }
  auto gradFunc = [inverse](std::vector<Variable>& inputs, const Variable& gradOutput) {
    inputs[0].addGrad(Variable(reorderTensor(gradOutput.tensor(), inverse), false));
  };
  return Variable(reorderTensor(input.tensor(), perm), {input}, gradFunc);
}

Variable linear(const Variable& input, const Variable& weight) {
  return linear(input, weight, Variable());
}

Variable linear(const Variable& input, const Variable& weight, const Variable& bias) {
  dtypesMatch("linear", {&input, &weight, &bias});
  if (weight.tensor().ndim() != 2 || input.tensor().ndim() < 1 ||
      input.tensor().dim(0) != weight.tensor().dim(1))
    throw std::invalid_argument("linear: weight must be [out, in] and input [in, ...]");
  const int tag = tagOf(input.type(), "linear");
  const Dim out = weight.tensor().dim(0), in = weight.tensor().dim(1);
  const Dim frames = input.tensor().elements() / in;
  std::vector<Dim> oshape = input.shape().get();
  oshape[0] = out;
  const bool hasBias = bias.tensor().elements() > 0;
  if (hasBias && bias.tensor().elements() != out)
    throw std::invalid_argument("linear: bias must have one element per output feature");
  // the tiled bias is added in fp32 inside the product (Functions.cpp:1267-1272)
  const Tensor b32 = hasBias ? bias.tensor().astype(dtype::f32) : Tensor();
  detail::OpScope scope("linear");
  Tensor output(Shape(oshape), input.type());
  check(flhip_matmul(weight.tensor().device(), input.tensor().device(), output.device(), (int32_t)out,
                     (int32_t)frames, (int32_t)in, 0, 0, static_cast<const float*>(b32.device()), tag,
                     hipBackendStream()));
  if (scope.on()) scope.done({input.tensor(), weight.tensor(), b32}, {output}, {out, in, frames});
  auto gradFunc = [hasBias, tag, out, in, frames](std::vector<Variable>& inputs,
                                                  const Variable& gradOutput) {
    // Functions.cpp:1276-1303
    detail::OpScope scope("linearBackward");
    auto& x = inputs[0];
    auto& wt = inputs[1];
    const void* g = gradOutput.tensor().device();
    Tensor dxT, dwT, dbT;
    if (hasBias && inputs[2].isCalcGrad()) {
      Tensor db(inputs[2].shape(), dtype::f32);
      const size_t wsBytes = flhip_sum_columns_workspace_bytes((int32_t)out, (int32_t)frames, tag);
      Tensor ws = wsBytes ? Tensor({(Dim)wsBytes}, dtype::u8) : Tensor();
      check(flhip_sum_columns_ws(g, static_cast<float*>(db.device()), (int32_t)out, (int32_t)frames, tag, ws.device(),
                                 wsBytes, hipBackendStream()));
      dbT = db;
    }
    if (x.isCalcGrad()) {
      Tensor dx(x.shape(), x.type());
      check(flhip_matmul(wt.tensor().device(), g, dx.device(), (int32_t)in, (int32_t)frames,
                         (int32_t)out, 1, 0, nullptr, tag, hipBackendStream()));
      dxT = dx;
    }
    if (wt.isCalcGrad()) {
      Tensor dw(wt.shape(), wt.type());
      // few tiles over a long contraction (the frames): with a workspace the library cuts it into slices
      const size_t wsBytes = flhip_matmul_workspace_bytes((int32_t)out, (int32_t)in, (int32_t)frames, 0, 1, tag);
      Tensor ws = wsBytes ? Tensor({(Dim)wsBytes}, dtype::u8) : Tensor();
      check(flhip_matmul_ws(g, x.tensor().device(), dw.device(), (int32_t)out, (int32_t)in,
                            (int32_t)frames, 0, 1, nullptr, tag, ws.device(), wsBytes, hipBackendStream()));
      dwT = dw;
    }
    // event: inputs {gradOutput, input, weight}, outputs {dx, dw, db (each may be empty)}, ints {out, in, frames}
    if (scope.on()) scope.done({gradOutput.tensor(), x.tensor(), wt.tensor()}, {dxT, dwT, dbT}, {out, in, frames});
    if (!dbT.isEmpty()) inputs[2].addGrad(Variable(dbT.astype(inputs[2].type()), false));
    if (!dxT.isEmpty()) x.addGrad(Variable(dxT, false));
    if (!dwT.isEmpty()) wt.addGrad(Variable(dwT, false));
  };
  if (hasBias) return Variable(output, {input, weight, bias}, gradFunc);
  return Variable(output, {input, weight}, gradFunc);
}

Variable logSoftmax(const Variable& input, int dim) {
  if (dim != 0) throw std::invalid_argument("logSoftmax: only dimension 0 is supported by this backend");
  const int tag = tagOf(input.type(), "logSoftmax");
  const Dim classes = input.tensor().dim(0), cols = input.tensor().elements() / classes;
  detail::OpScope scope("logSoftmax");
  Tensor result(input.shape(), input.type());
  check(flhip_logsoftmax_fwd(input.tensor().device(), result.device(), (int32_t)classes, (int32_t)cols,
                             tag, hipBackendStream()));
  if (scope.on()) scope.done({input.tensor()}, {result}, {classes, cols});
  auto gradFunc = [result, tag, classes, cols](std::vector<Variable>& inputs,
                                               const Variable& gradOutput) {
    // gradOutput - exp(result) * sum(gradOutput) (Functions.cpp:1061-1066)
    detail::OpScope scope("logSoftmaxBackward");
    Tensor g(result.shape(), result.type());
    check(flhip_logsoftmax_bwd(gradOutput.tensor().device(), result.device(), g.device(),
                               (int32_t)classes, (int32_t)cols, tag, hipBackendStream()));
    if (scope.on()) scope.done({gradOutput.tensor(), result}, {g}, {classes, cols});
    inputs[0].addGrad(Variable(g.astype(inputs[0].type()), false));
  };
  return Variable(result, {input}, gradFunc);
}

Variable categoricalCrossEntropy(const Variable& input, const Variable& targets, ReduceMode reduction,
                                 int ignoreIndex) {
  // Functions.cpp:1086-1098
  if (input.tensor().ndim() != targets.tensor().ndim() + 1)
    throw std::invalid_argument("dimension mismatch in categorical cross entropy: "
                                "target must have one fewer dimension than input");
  for (int i = 1; i < input.tensor().ndim(); ++i)
    if (input.tensor().dim(i) != targets.tensor().dim(i - 1))
      throw std::invalid_argument("dimension mismatch in categorical cross entropy");
  if (targets.type() != dtype::s32)
    throw std::invalid_argument("categoricalCrossEntropy: targets must be s32 on this backend");
  const int tag = tagOf(input.type(), "categoricalCrossEntropy");
  const Dim C = input.tensor().dim(0), X = targets.tensor().elements();
  detail::OpScope scope("categoricalCrossEntropy");
  Tensor stats(Shape({4}), dtype::f32);
  Tensor per = reduction == ReduceMode::NONE ? Tensor(targets.shape(), dtype::f32) : Tensor();
  check(flhip_cce_fwd(input.tensor().device(), static_cast<const int32_t*>(targets.tensor().device()),
                      static_cast<float*>(stats.device()), static_cast<float*>(per.device()),
                      (int32_t)C, (int32_t)X, ignoreIndex, tag, hipBackendStream()));
  // the reference reads a device scalar here too (:1100-1108)
  const std::vector<float> st = stats.toHostVector();
  if (st[2] != 0.f)
    throw std::invalid_argument("target contains elements out of valid range [0, num_categories) "
                                "in categorical cross entropy");
  Tensor result;
  if (reduction == ReduceMode::NONE) {
    result = per;
  } else {
    const float v = reduction == ReduceMode::MEAN ? st[3] : st[0];
    result = Tensor::fromHost(Shape({1}), dtype::f32, &v);
  }
  if (scope.on()) scope.done({input.tensor(), targets.tensor()}, {result, stats}, {C, X, (int)reduction, ignoreIndex});
  const Shape inShape = input.shape();
  const dtype inType = input.type();
  const Tensor tg = targets.tensor();
  auto gradFunc = [stats, tg, inShape, inType, tag, C, X, reduction, ignoreIndex](
                      std::vector<Variable>& inputs, const Variable& gradOutput) {
    // tile(grad / denominator) * mask (Functions.cpp:1131-1150)
    detail::OpScope scope("categoricalCrossEntropyBackward");
    Tensor g(inShape, inType);
    const Tensor go = gradOutput.tensor().astype(dtype::f32);
    check(flhip_cce_bwd(static_cast<const float*>(go.device()),
                        static_cast<const int32_t*>(tg.device()),
                        static_cast<const float*>(stats.device()), g.device(), (int32_t)C, (int32_t)X,
                        (int)reduction, ignoreIndex, tag, hipBackendStream()));
    if (scope.on()) scope.done({go, tg, stats}, {g}, {C, X, (int)reduction, ignoreIndex});
    inputs[0].addGrad(Variable(g, false));
  };
  return Variable(result, {input, targets}, gradFunc);
}

}  // namespace fl
