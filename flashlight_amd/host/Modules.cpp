#include "Modules.h"

#include <memory>

#include "flhip.h"

#include <algorithm>
#include <cmath>
#include <random>
#include <sstream>

namespace fl {

// ---- initialisation --------------------------------------------------------------------
namespace {
std::mt19937_64& generator() {
  static std::mt19937_64 gen(0);
  return gen;
}
Tensor fromFloats(const Shape& shape, dtype type, const std::vector<float>& v) {
  if (type != dtype::f32 && type != dtype::bf16 && type != dtype::f16)
    throw std::invalid_argument("initialisation: f32, bf16 and f16 only");
  Tensor t = Tensor::fromVector(shape, v);
  return type == dtype::f32 ? t : t.astype(type);
}
}  // namespace

void setSeed(unsigned long long seed) { generator().seed(seed); }
unsigned long long nextSeed() { return generator()(); }

Variable constant(double val, const Shape& shape, dtype type, bool calcGrad) {
  return Variable(fromFloats(shape, type, std::vector<float>((size_t)shape.elements(), (float)val)),
                  calcGrad);
}

Variable uniform(const Shape& shape, double min, double max, dtype type, bool calcGrad) {
  // (max - min) * rand + min (Init.cpp:22-26)
  std::uniform_real_distribution<double> d(0.0, 1.0);
  std::vector<float> v((size_t)shape.elements());
  for (auto& x : v) x = (float)((max - min) * d(generator()) + min);
  return Variable(fromFloats(shape, type, v), calcGrad);
}

Variable kaimingUniform(const Shape& shape, int fanIn, dtype type, bool calcGrad) {
  // Init.cpp:33-40
  const double stdv = std::sqrt(1.0 / (double)fanIn);
  const double limit = std::sqrt(3.0) * stdv;
  return uniform(shape, -limit, limit, type, calcGrad);
}

Variable normal(const Shape& shape, double stdv, double mean, dtype type, bool calcGrad) {
  // stdv * randn + mean (Init.cpp:28-30)
  std::normal_distribution<double> d(0.0, 1.0);
  std::vector<float> v((size_t)shape.elements());
  for (auto& x : v) x = (float)(stdv * d(generator()) + mean);
  return Variable(fromFloats(shape, type, v), calcGrad);
}

Variable kaimingNormal(const Shape& shape, int fanIn, dtype type, bool calcGrad) {
  return normal(shape, std::sqrt(1.0 / (double)fanIn), 0.0, type, calcGrad);   // Init.cpp:42-48
}

Variable glorotUniform(const Shape& shape, int fanIn, int fanOut, dtype type, bool calcGrad) {
  const double limit = std::sqrt(3.0) * std::sqrt(2.0 / (double)(fanIn + fanOut));   // Init.cpp:50-58
  return uniform(shape, -limit, limit, type, calcGrad);
}

Variable glorotNormal(const Shape& shape, int fanIn, int fanOut, dtype type, bool calcGrad) {
  return normal(shape, std::sqrt(2.0 / (double)(fanIn + fanOut)), 0.0, type, calcGrad);   // Init.cpp:60-68
}

// ---- Module ----------------------------------------------------------------------------
Variable Module::param(int position) const {
  if (!(position >= 0 && position < (int)params_.size()))
    throw std::out_of_range("Module param index out of range");
  return params_[position];
}

void Module::setParams(const Variable& var, int position) {
  if (!(position >= 0 && position < (int)params_.size()))
    throw std::out_of_range("Module param index out of range");
  params_[position] = var;
}

void Module::train() {
  train_ = true;
  for (auto& p : params_) p.setCalcGrad(true);
}

void Module::eval() {
  train_ = false;
  for (auto& p : params_) p.setCalcGrad(false);
}

void Module::zeroGrad() {
  for (auto& p : params_) p.zeroGrad();
}

std::vector<Variable> UnaryModule::forward(const std::vector<Variable>& inputs) {
  if (inputs.size() != 1) throw std::invalid_argument("UnaryModule expects only one input");
  return {forward(inputs[0])};
}

std::vector<Variable> BinaryModule::forward(const std::vector<Variable>& inputs) {
  if (inputs.size() != 2) throw std::invalid_argument("BinaryModule expects two inputs");
  return {forward(inputs[0], inputs[1])};
}

// ---- Container / Sequential ---------------------------------------------------------------
void Container::train() {
  train_ = true;
  for (auto& m : modules_) m->train();
}

void Container::eval() {
  train_ = false;
  for (auto& m : modules_) m->eval();
}

void Container::setParams(const Variable& var, int position) {
  Module::setParams(var, position);
  for (const auto& c : childParamIdx_)
    if (c.position == position) modules_[c.module]->setParams(var, c.index);
}

std::vector<Variable> Container::castParams() const {
  std::vector<Variable> all;
  for (const auto& m : modules_) {
    const auto p = m->castParams();
    all.insert(all.end(), p.begin(), p.end());
  }
  return all;
}

std::vector<Variable> Sequential::forward(const std::vector<Variable>& inputs) {
  // activations in another type than the fp32 parameters: every module's casts in one launch
  std::unique_ptr<detail::ParamCastScope> casts;
  if (!inputs.empty() && !inputs[0].isEmpty() && inputs[0].type() != dtype::f32)
    casts.reset(new detail::ParamCastScope(castParams(), inputs[0].type()));
  auto output = inputs;
  for (auto& m : modules_) output = m->forward(output);
  return output;
}

Variable Sequential::forward(const Variable& input) {
  std::unique_ptr<detail::ParamCastScope> casts;
  if (!input.isEmpty() && input.type() != dtype::f32)
    casts.reset(new detail::ParamCastScope(castParams(), input.type()));
  std::vector<Variable> output = {input};
  for (auto& m : modules_) output = m->forward(output);
  if (output.size() != 1) throw std::invalid_argument("Module output size is not 1");
  return output.front();
}

std::string Sequential::prettyString() const {
  std::ostringstream ss;
  ss << "Sequential [input";
  for (size_t i = 0; i < modules_.size(); ++i) ss << " -> (" << i << ")";
  ss << " -> output]";
  for (size_t i = 0; i < modules_.size(); ++i) ss << "\n\t(" << i << "): " << modules_[i]->prettyString();
  return ss.str();
}

// ---- Conv2D ----------------------------------------------------------------------------
Conv2D::Conv2D(int nin, int nout, int wx, int wy, int sx, int sy, IntOrPadMode px, IntOrPadMode py,
               int dx, int dy, bool bias, int groups)
    : nIn_(nin), nOut_(nout), xFilter_(wx), yFilter_(wy), xStride_(sx), yStride_(sy), xPad_(px.padVal),
      yPad_(py.padVal), xDilation_(dx), yDilation_(dy), bias_(bias), groups_(groups) {
  if (groups <= 0 || nin % groups != 0)
    throw std::invalid_argument("Conv2D: input channels must divide into the groups");
  const int fanIn = xFilter_ * yFilter_ * nIn_ / groups_;
  auto wt = kaimingUniform(Shape({xFilter_, yFilter_, nIn_ / groups_, nOut_}), fanIn, dtype::f32, true);
  if (bias_) {
    const double bound = std::sqrt(1.0 / fanIn);
    params_ = {wt, uniform(Shape({1, 1, nOut_, 1}), -bound, bound, dtype::f32, true)};
  } else {
    params_ = {wt};
  }
}

Conv2D::Conv2D(const Variable& w, int sx, int sy, IntOrPadMode px, IntOrPadMode py, int dx, int dy,
               int groups)
    : UnaryModule({w}), nIn_((int)w.dim(2) * groups), nOut_((int)w.dim(3)), xFilter_((int)w.dim(0)),
      yFilter_((int)w.dim(1)), xStride_(sx), yStride_(sy), xPad_(px.padVal), yPad_(py.padVal),
      xDilation_(dx), yDilation_(dy), bias_(false), groups_(groups) {}

Conv2D::Conv2D(const Variable& w, const Variable& b, int sx, int sy, IntOrPadMode px, IntOrPadMode py,
               int dx, int dy, int groups)
    : UnaryModule({w, b}), nIn_((int)w.dim(2) * groups), nOut_((int)w.dim(3)), xFilter_((int)w.dim(0)),
      yFilter_((int)w.dim(1)), xStride_(sx), yStride_(sy), xPad_(px.padVal), yPad_(py.padVal),
      xDilation_(dx), yDilation_(dy), bias_(true), groups_(groups) {
  if (b.ndim() < 3 || b.dim(2) != w.dim(3))
    throw std::invalid_argument("output channel dimension mismatch between Conv2D weight and bias");
  if (b.elements() != b.dim(2))
    throw std::invalid_argument("only 3rd dimension of Conv2D bias may be non-singleton");
}

Variable Conv2D::forward(const Variable& input) {
  const int px = derivePadding((int)input.dim(0), xFilter_, xStride_, xPad_, xDilation_);
  const int py = derivePadding((int)input.dim(1), yFilter_, yStride_, yPad_, yDilation_);
  if (!(px >= 0 && py >= 0)) throw std::invalid_argument("invalid padding for Conv2D");
  if (bias_)
    return conv2d(input, params_[0].astype(input.type()), params_[1].astype(input.type()), xStride_,
                  yStride_, px, py, xDilation_, yDilation_, groups_, benchmarks_);
  return conv2d(input, params_[0].astype(input.type()), xStride_, yStride_, px, py, xDilation_,
                yDilation_, groups_, benchmarks_);
}

namespace {
std::string padString(int p) {
  return p == static_cast<int>(PaddingMode::SAME) ? std::string("SAME") : std::to_string(p);
}
}  // namespace

std::string Conv2D::prettyString() const {
  std::ostringstream ss;
  ss << "Conv2D (" << nIn_ << "->" << nOut_ << ", " << xFilter_ << "x" << yFilter_ << ", " << xStride_
     << "," << yStride_ << ", " << padString(xPad_) << "," << padString(yPad_) << ", " << xDilation_
     << ", " << yDilation_ << ")" << (bias_ ? " (with bias)" : " (without bias)");
  return ss.str();
}

// ---- Padding, WeightNorm ------------------------------------------------------------------
std::string Padding::prettyString() const {
  std::ostringstream ss;
  ss << "Padding (" << val_ << ", { ";
  for (const auto& p : pad_) ss << "(" << p.first << ", " << p.second << "), ";
  ss << "})";
  return ss.str();
}

WeightNorm::WeightNorm(ModulePtr module, int dim) : module_(std::move(module)), dim_(dim) {
  if (!module_) throw std::invalid_argument("WeightNorm: null module");
  const auto mp = module_->params();
  if (mp.size() != 1 && mp.size() != 2) throw std::invalid_argument("WeightNorm only supports Linear and Conv2D");
  const Variable& v = mp[0];
  if (dim_ < 0 || dim_ > v.ndim()) throw std::invalid_argument("invalid dimension for WeightNorm");   // WeightNorm.cpp:36-38
  Variable g(rowNorm(v.tensor(), dim_), true);                                                          // :68-72
  params_ = mp.size() == 2 ? std::vector<Variable>{v, g, mp[1]} : std::vector<Variable>{v, g};
  computeWeight();
}

void WeightNorm::computeWeight() { module_->setParams(weightNorm(params_[0], params_[1], dim_), 0); }   // :45-66

void WeightNorm::setParams(const Variable& var, int position) {
  Module::setParams(var, position);
  // :84-93: the wrapped module keeps copies, not pointers
  if (position == 2)
    module_->setParams(var, 1);
  else if (position <= 1)
    computeWeight();
}

std::vector<Variable> WeightNorm::forward(const std::vector<Variable>& inputs) {
  if (train_) computeWeight();                                                                         // :95-100
  return module_->forward(inputs);
}

void WeightNorm::train() {
  Module::train();
  module_->train();
}

void WeightNorm::eval() {
  Module::eval();
  module_->eval();
  computeWeight();
}

std::string WeightNorm::prettyString() const {
  std::ostringstream ss;
  ss << "WeightNorm (" << module_->prettyString() << ", " << dim_ << ")";
  return ss.str();
}

// ---- AsymmetricConv1D, TDSBlock (flashlight/fl/contrib/modules) -------------------------
AsymmetricConv1D::AsymmetricConv1D(int nin, int nout, int wx, int sx, IntOrPadMode px, float futurePart, int dx,
                                   bool bias, int groups)
    : Conv2D(nin, nout, wx, 1, sx, 1, px, 0, dx, 1, bias, groups), futurePart_(futurePart) {
  // AsymmetricConv1D.cpp:16-25
  if (xPad_ != static_cast<int>(PaddingMode::SAME) && xPad_ != 0)
    throw std::invalid_argument("AsymmetricConv1D: invalid xPad_, now supports only '0' or 'SAME' ");
  if (futurePart_ < 0 || futurePart_ > 1)
    throw std::invalid_argument("AsymmetricConv1D: invalid futurePart_, should be in [0, 1]");
}

Variable AsymmetricConv1D::forward(const Variable& input) {
  // AsymmetricConv1D.cpp:64-104
  const int px = derivePadding((int)input.dim(0), xFilter_, xStride_, xPad_, xDilation_);
  if (!(px >= 0)) throw std::invalid_argument("invalid padding for AsymmetricConv1D");
  const int cutPx = (int)(std::abs(2 * (0.5 - futurePart_)) * px);
  const int asymmetryPx = px + cutPx;
  Variable output =
      bias_ ? conv2d(input, params_[0].astype(input.type()), params_[1].astype(input.type()), xStride_, yStride_,
                     asymmetryPx, 0, xDilation_, yDilation_, groups_, benchmarks_)
            : conv2d(input, params_[0].astype(input.type()), xStride_, yStride_, asymmetryPx, 0, xDilation_, yDilation_,
                     groups_, benchmarks_);
  if (cutPx == 0) return output;
  if (futurePart_ < 0.5) return narrow(output, 0, 0, output.dim(0) - 2 * cutPx);
  if (futurePart_ > 0.5) return narrow(output, 0, 2 * cutPx, output.dim(0) - 2 * cutPx);
  return output;
}

std::string AsymmetricConv1D::prettyString() const { return "AsymmetricConv1D (" + Conv2D::prettyString() + ")"; }

TDSBlock::TDSBlock(int channels, int kernelSize, int width, double dropout, int innerLinearDim, int rightPadding,
                   bool lNormIncludeTime) {
  // TDSBlock.cpp:13-67
  Sequential conv;
  int convPadding = static_cast<int>(PaddingMode::SAME);
  if (rightPadding != -1) {
    const int totalPadding = kernelSize - 1;
    if (rightPadding > totalPadding)
      throw std::invalid_argument("right padding exceeds the 'SAME' padding required for TDSBlock");
    conv.add(Padding({std::pair<int, int>{totalPadding - rightPadding, rightPadding}}, 0.0));
    convPadding = 0;
  }
  conv.add(Conv2D(channels, channels, kernelSize, 1, 1, 1, convPadding, 0));
  conv.add(ReLU());
  conv.add(Dropout(dropout));
  const int linearDim = channels * width;
  if (innerLinearDim == 0) innerLinearDim = linearDim;
  Sequential fc;
  fc.add(Reorder(Shape({2, 1, 0, 3})));
  fc.add(View(Shape({linearDim, -1, 1, 0})));
  fc.add(Linear(linearDim, innerLinearDim));
  fc.add(ReLU());
  if (dropout > 0) fc.add(Dropout(dropout));
  fc.add(Linear(innerLinearDim, linearDim));
  fc.add(View(Shape({channels, width, -1, 0})));
  fc.add(Reorder(Shape({2, 1, 0, 3})));
  if (dropout > 0) fc.add(Dropout(dropout));
  const std::vector<int> axes = lNormIncludeTime ? std::vector<int>{0, 1, 2} : std::vector<int>{1, 2};
  add(std::move(conv));
  add(LayerNorm(axes));
  add(std::move(fc));
  add(LayerNorm(axes));
}

std::vector<Variable> TDSBlock::forward(const std::vector<Variable>& inputs) {
  // TDSBlock.cpp:69-75
  if (inputs.size() != 1) throw std::invalid_argument("TDSBlock expects one input");
  Variable out = inputs[0];
  out = module(0)->forward({out})[0].astype(out.type()) + out;
  out = module(1)->forward({out})[0];
  out = module(2)->forward({out})[0].astype(out.type()) + out;
  return module(3)->forward({out});
}

std::string TDSBlock::prettyString() const {
  // TDSBlock.cpp:77-91
  std::ostringstream ss;
  const Variable convW = param(0), linW = param(4);
  const int kw = (int)convW.dim(0), c = (int)convW.dim(2);
  const int w = (int)linW.dim(0) / c, l = (int)linW.dim(1), l2 = (int)linW.dim(0);
  ss << "Time-Depth Separable Block (" << kw << ", " << w << ", " << c << ") [" << l << " -> " << l2 << " -> " << l << "]";
  return ss.str();
}

// ---- Residual (flashlight/fl/contrib/modules/Residual.cpp) --------------------------------
void Residual::addScale(int beforeLayer, float scale) {
  const int nLayers = (int)modules_.size() - (int)projectionsIndices_.size();
  if (beforeLayer < 1 || beforeLayer > nLayers + 1)
    throw std::invalid_argument("Residual: invalid layer index " + std::to_string(beforeLayer) +
                                " before which apply the scaling");
  if (scales_.find(beforeLayer - 1) != scales_.end())
    throw std::invalid_argument("Residual: scaling before layer " + std::to_string(beforeLayer) +
                                " was already added; adding only once is allowed");
  scales_[beforeLayer - 1] = scale;
}

void Residual::checkShortcut(int fromLayer, int toLayer) {
  const int nLayers = (int)modules_.size() - (int)projectionsIndices_.size();
  if (fromLayer < 0 || fromLayer >= nLayers || toLayer <= 0 || toLayer > nLayers + 2 || toLayer - fromLayer <= 1)
    throw std::invalid_argument("Residual: invalid skip connection; check fromLayer=" + std::to_string(fromLayer) +
                                " and toLayer=" + std::to_string(toLayer) +
                                " parameters. They are out of range of added layers");
  const auto it = shortcut_.find(toLayer - 1);
  if (it != shortcut_.end() && it->second.find(fromLayer) != it->second.end())
    throw std::invalid_argument("Residual: skip connection for fromLayer " + std::to_string(fromLayer) + " to toLayer " +
                                std::to_string(toLayer) + " is already added");
}

void Residual::addShortcut(int fromLayer, int toLayer) {
  checkShortcut(fromLayer, toLayer);
  shortcut_[toLayer - 1].insert({fromLayer, -1});
}

void Residual::addShortcut(int fromLayer, int toLayer, ModulePtr projection) {
  checkShortcut(fromLayer, toLayer);
  Container::add(std::move(projection));
  shortcut_[toLayer - 1].insert({fromLayer, (int)modules_.size() - 1});
  projectionsIndices_.insert((int)modules_.size() - 1);
}

Variable Residual::applyScale(const Variable& input, int layerIndex) {
  // Residual.cpp:69-73 multiplies by 1 where no scale was given: the same values
  const auto it = scales_.find(layerIndex);
  return it == scales_.end() ? input : input * (double)it->second;
}

std::vector<Variable> Residual::forward(const std::vector<Variable>& inputs) {
  if (inputs.size() != 1) throw std::invalid_argument("Residual module expects only one input");
  return {forward(inputs[0])};
}

Variable Residual::forward(const Variable& input) {
  // Residual.cpp:82-124
  Variable output = input;
  const int nLayers = (int)modules_.size() - (int)projectionsIndices_.size();
  std::vector<Variable> outputs((size_t)nLayers + 1);
  outputs[0] = input;
  auto addShortcuts = [&](int layerIndex) {
    const auto it = shortcut_.find(layerIndex);
    if (it == shortcut_.end()) return;
    for (const auto& sc : it->second) {
      Variable connectionOut = outputs[(size_t)sc.first];
      if (sc.second != -1) connectionOut = modules_[(size_t)sc.second]->forward({outputs[(size_t)sc.first]}).front();
      output = output + connectionOut.astype(output.type());
    }
  };
  int moduleIndex = 0;
  for (int layerIndex = 0; layerIndex < nLayers; ++layerIndex, ++moduleIndex) {
    while (projectionsIndices_.count(moduleIndex)) ++moduleIndex;
    addShortcuts(layerIndex);
    output = modules_[(size_t)moduleIndex]->forward({applyScale(output, layerIndex)}).front();
    outputs[(size_t)layerIndex + 1] = output;
  }
  addShortcuts(nLayers);
  return applyScale(output, nLayers);
}

std::string Residual::prettyString() const {
  std::ostringstream ss;
  const int nLayers = (int)modules_.size() - (int)projectionsIndices_.size();
  ss << "Residual (" << nLayers << " layers";
  for (const auto& end : shortcut_)
    for (const auto& sc : end.second) {
      ss << "; skip " << sc.first << " -> " << end.first + 1;
      if (sc.second != -1) ss << " through " << modules_[(size_t)sc.second]->prettyString();
    }
  for (const auto& sc : scales_) ss << "; scale " << sc.second << " before " << sc.first + 1;
  ss << ")";
  return ss.str();
}

// ---- Pool2D ----------------------------------------------------------------------------
Pool2D::Pool2D(int wx, int wy, int sx, int sy, IntOrPadMode px, IntOrPadMode py, PoolingMode mode)
    : xFilter_(wx), yFilter_(wy), xStride_(sx), yStride_(sy), xPad_(px.padVal), yPad_(py.padVal),
      mode_(mode) {}

Variable Pool2D::forward(const Variable& input) {
  const int px = derivePadding((int)input.dim(0), xFilter_, xStride_, xPad_, 1);
  const int py = derivePadding((int)input.dim(1), yFilter_, yStride_, yPad_, 1);
  if (!(px >= 0 && py >= 0)) throw std::invalid_argument("invalid padding for Pool2D");
  return pool2d(input, xFilter_, yFilter_, xStride_, yStride_, px, py, mode_);
}

std::string Pool2D::prettyString() const {
  std::ostringstream ss;
  ss << "Pool2D"
     << (mode_ == PoolingMode::MAX ? "-max"
                                   : mode_ == PoolingMode::AVG_EXCLUDE_PADDING ? "-avg(without pad)"
                                                                               : "-avg(with pad)")
     << " (" << xFilter_ << "x" << yFilter_ << ", " << xStride_ << "," << yStride_ << ", "
     << padString(xPad_) << "," << padString(yPad_) << ")";
  return ss.str();
}

// ---- BatchNorm -------------------------------------------------------------------------
BatchNorm::BatchNorm(int featAxis, int featSize, double momentum, double eps, bool affine,
                     bool trackStats)
    : BatchNorm(std::vector<int>(1, featAxis), featSize, momentum, eps, affine, trackStats) {}

BatchNorm::BatchNorm(const std::vector<int>& featAxis, int featSize, double momentum, double eps,
                     bool affine, bool trackStats)
    : featAxis_(featAxis), featSize_(featSize), momentum_(momentum), epsilon_(eps), affine_(affine),
      trackStats_(trackStats) {
  // BatchNorm.cpp:100-112
  if (trackStats_) {
    runningMean_ = constant(0.0, Shape({featSize_}), dtype::f32, false);
    runningVar_ = constant(1.0, Shape({featSize_}), dtype::f32, false);
  }
  if (affine_)
    params_ = {uniform(Shape({featSize_}), 0.0, 1.0, dtype::f32, true),
               constant(0.0, Shape({featSize_}), dtype::f32, true)};
}

Variable BatchNorm::forward(const Variable& input) {
  // BatchNorm.cpp:74-98
  double avgFactor = 0.0;
  if (train_ && trackStats_) {
    ++numBatchesTracked_;
    avgFactor = momentum_ < 0 ? 1.0 / numBatchesTracked_ : momentum_;
  }
  // parameters stay f32 for 16-bit inputs (the reference does this for f16)
  const Variable none(Tensor(), false);
  return batchnorm(input, params_.empty() ? none : params_[0], params_.empty() ? none : params_[1],
                   runningMean_, runningVar_, featAxis_, train_ || !trackStats_, avgFactor, epsilon_);
}

Variable BatchNorm::forwardRelu(const Variable& input, const Variable& residual) {
  if (!(train_ || !trackStats_)) {
    // inference with running statistics: no fused kernel, the composition is exact
    Variable y = forward(input);
    return relu(residual.isEmpty() ? y : y + residual);
  }
  double avgFactor = 0.0;
  if (train_ && trackStats_) {
    ++numBatchesTracked_;
    avgFactor = momentum_ < 0 ? 1.0 / numBatchesTracked_ : momentum_;
  }
  const Variable none(Tensor(), false);
  return detail::batchnormRelu(input, params_.empty() ? none : params_[0], params_.empty() ? none : params_[1],
                               runningMean_, runningVar_, featAxis_, avgFactor, epsilon_, residual);
}

std::string BatchNorm::prettyString() const {
  std::ostringstream ss;
  ss << "BatchNorm ( axis : { ";
  for (int a : featAxis_) ss << a << " ";
  ss << "}, size : " << featSize_ << " )";
  return ss.str();
}

// ---- LayerNorm -------------------------------------------------------------------------
namespace {
constexpr int kLnExpectedNumDims = 4;
}

LayerNorm::LayerNorm(int axis, double eps, bool affine, int axisSize)
    : LayerNorm(std::vector<int>({axis}), eps, affine, axisSize) {}

LayerNorm::LayerNorm(const std::vector<int>& axis, double eps, bool affine, int axisSize)
    : axis_(axis), epsilon_(eps), affine_(affine), axisSize_(axisSize) {
  for (int d = 0; d < kLnExpectedNumDims; ++d)
    if (std::find(axis.begin(), axis.end(), d) == axis.end()) axisComplement_.push_back(d);
  if (axisComplement_.empty()) throw std::invalid_argument("LayerNorm: no axis left to batch over");
  std::sort(axis_.begin(), axis_.end());
  if (affine_) {
    const int paramDim = axisSize_ == kLnVariableAxisSize ? 1 : axisSize_;
    params_ = {constant(1.0, Shape({paramDim}), dtype::f32, true),
               constant(0.0, Shape({paramDim}), dtype::f32, true)};
  }
}

Variable LayerNorm::forward(const Variable& in) {
  // LayerNorm.cpp:42-131
  Variable input = in;
  if (input.ndim() < kLnExpectedNumDims) {
    std::vector<Dim> s = in.shape().get();
    while ((int)s.size() < kLnExpectedNumDims) s.push_back(1);
    input = moddims(in, Shape(s));
  } else if (input.ndim() > kLnExpectedNumDims) {
    throw std::invalid_argument("LayerNorm::forward - input must be " +
                                std::to_string(kLnExpectedNumDims) + " or fewer dimensions.");
  }
  const int maxAxis = *std::max_element(axisComplement_.begin(), axisComplement_.end());
  const int minAxis = *std::min_element(axisComplement_.begin(), axisComplement_.end());
  bool axesContinuous = (int)axisComplement_.size() == maxAxis - minAxis + 1;
  // per-element parameters over normalised axes that are not contiguous take the reorder too: the
  // broadcast kernel wants them side by side, and the two reorders cancel
  if (affine_ && axisSize_ != kLnVariableAxisSize && axis_.back() - axis_.front() + 1 != (int)axis_.size())
    axesContinuous = false;
  // a complement that is not contiguous: reorder so that the normalised axes lead and the
  // complement follows, batch-normalise over the trailing axes, reorder back (:63-86, 98-108)
  Variable inputToBn = input;
  std::vector<int> inNormAxes = axisComplement_, normAxes = axis_;
  std::vector<Dim> reorderDims, restoreDims((size_t)input.ndim());
  if (!axesContinuous) {
    for (int d : axis_) reorderDims.push_back(d);
    inNormAxes.clear();
    for (int d : axisComplement_) {
      inNormAxes.push_back((int)reorderDims.size());
      reorderDims.push_back(d);
    }
    for (size_t i = 0; i < reorderDims.size(); ++i) restoreDims[(size_t)reorderDims[i]] = (Dim)i;
    inputToBn = reorder(input, Shape(reorderDims));
    for (size_t i = 0; i < axis_.size(); ++i) normAxes[i] = (int)i;
  }
  Variable dummyInMean, dummyInVar;
  const Variable none(Tensor(), false);
  Variable output = batchnorm(inputToBn, none, none, dummyInMean, dummyInVar, inNormAxes, true, 0.0,
                              epsilon_);
  // The scale and shift broadcast one parameter element per position along the normalised
  // axes (:110-128).  After a reorder they are applied before reordering back: the
  // normalised axes lead there, in the parameters' own order, so the broadcast is the
  // contiguous [outer][mid][inner] one; the result is the same as tiling over the restored
  // tensor.
  if (affine_) {
    const Variable weight = params_[0].astype(output.type());
    const Variable bias = params_[1].astype(output.type());
    if (axisSize_ == kLnVariableAxisSize) {
      output = detail::affine(output, weight, bias, 1, 1, output.elements(), true);
    } else {
      if (normAxes.empty() || normAxes.back() - normAxes.front() + 1 != (int)normAxes.size())
        throw std::invalid_argument("LayerNorm: per-element parameters need contiguous normalised axes");
      Dim inner = 1, mid = 1, outer = 1;
      for (int d = 0; d < output.ndim(); ++d)
        (d < normAxes.front() ? inner : d <= normAxes.back() ? mid : outer) *= output.dim(d);
      if (mid != axisSize_)
        throw std::invalid_argument("[LayerNorm] Input size along the norm axis doesn't with axisSize.");
      output = detail::affine(output, weight, bias, outer, mid, inner, false);
    }
  }
  if (!axesContinuous) output = reorder(output, Shape(restoreDims));
  return moddims(output, in.shape());
}

std::string LayerNorm::prettyString() const {
  std::ostringstream ss;
  ss << "LayerNorm ( axis : { ";
  for (int a : axis_) ss << a << " ";
  ss << "} , size : " << axisSize_ << ")";
  return ss.str();
}

// ---- RNN -------------------------------------------------------------------------------
int64_t detail::getNumRnnParams(int inputSize, int hiddenSize, int numLayers, RnnMode mode, bool bidirectional) {
  flhip_rnn_desc d{};
  d.input_size = inputSize; d.hidden_size = hiddenSize; d.num_layers = numLayers;
  d.bidirectional = bidirectional ? 1 : 0; d.mode = (int32_t)mode; d.seq_len = 1; d.batch = 1; d.dtype = FLHIP_F32;
  const size_t n = flhip_rnn_param_count(&d);
  if (n == 0) throw std::invalid_argument("RNN: invalid sizes");
  return (int64_t)n;
}

RNN::RNN(int inputSize, int hiddenSize, int numLayers, RnnMode mode, bool bidirectional, float dropProb)
    : inputSize_(inputSize), hiddenSize_(hiddenSize), numLayers_(numLayers), mode_(mode),
      bidirectional_(bidirectional), dropProb_(dropProb) {
  const int64_t n = detail::getNumRnnParams(inputSize_, hiddenSize_, numLayers_, mode_, bidirectional_);
  const double stdv = std::sqrt(1.0 / (double)hiddenSize_);
  params_ = {uniform(Shape({(Dim)n}), -stdv, stdv, dtype::f32, true)};
}

std::vector<Variable> RNN::forward(const std::vector<Variable>& inputs) {
  if (inputs.empty() || inputs.size() > 3) throw std::invalid_argument("Invalid inputs size");
  const Variable& input = inputs[0];
  const Variable hiddenState = inputs.size() >= 2 ? inputs[1] : Variable();
  const Variable cellState = inputs.size() == 3 ? inputs[2] : Variable();
  const float dropProb = train_ ? dropProb_ : 0.f;
  auto res = rnn(input, hiddenState, cellState, params_[0].astype(input.type()), hiddenSize_, numLayers_, mode_,
                 bidirectional_, dropProb);
  std::vector<Variable> output(1, std::get<0>(res));
  if (inputs.size() >= 2) output.push_back(std::get<1>(res));
  if (inputs.size() == 3) output.push_back(std::get<2>(res));
  return output;
}

std::tuple<Variable, Variable> RNN::forward(const Variable& input, const Variable& hiddenState) {
  auto r = forward(std::vector<Variable>{input, hiddenState});
  return std::make_tuple(r[0], r[1]);
}

std::tuple<Variable, Variable, Variable> RNN::forward(const Variable& input, const Variable& hiddenState,
                                                      const Variable& cellState) {
  auto r = forward(std::vector<Variable>{input, hiddenState, cellState});
  return std::make_tuple(r[0], r[1], r[2]);
}

std::string RNN::prettyString() const {
  std::ostringstream ss;
  ss << (mode_ == RnnMode::RELU ? "RNN (relu)" : mode_ == RnnMode::TANH ? "RNN (tanh)" : mode_ == RnnMode::LSTM ? "LSTM" : "GRU");
  ss << " (" << inputSize_ << "->" << (bidirectional_ ? 2 * hiddenSize_ : hiddenSize_) << ")";
  if (numLayers_ > 1) ss << " (" << numLayers_ << "-layer)";
  if (bidirectional_) ss << " (bidirectional)";
  if (dropProb_ > 0) ss << " (dropout=" << dropProb_ << ")";
  return ss.str();
}

// ---- Linear ----------------------------------------------------------------------------
Linear::Linear(int inputSize, int outputSize, bool bias) : nIn_(inputSize), nOut_(outputSize), bias_(bias) {
  // Linear.cpp:62-74
  const int fanIn = nIn_;
  auto w = kaimingUniform(Shape({nOut_, nIn_}), fanIn, dtype::f32, true);
  if (bias_) {
    const double bound = std::sqrt(1.0 / fanIn);
    params_ = {w, uniform(Shape({nOut_}), -bound, bound, dtype::f32, true)};
  } else {
    params_ = {w};
  }
}

Linear::Linear(const Variable& w) : UnaryModule({w}), nIn_((int)w.dim(1)), nOut_((int)w.dim(0)), bias_(false) {}

Linear::Linear(const Variable& w, const Variable& b)
    : UnaryModule({w, b}), nIn_((int)w.dim(1)), nOut_((int)w.dim(0)), bias_(true) {
  if (b.dim(0) != w.dim(0)) throw std::invalid_argument("dimension mismatch between Linear weight and bias");
}

Variable Linear::forward(const Variable& input) {
  if (bias_) return linear(input, params_[0].astype(input.type()), params_[1].astype(input.type()));
  return linear(input, params_[0].astype(input.type()));
}

std::string Linear::prettyString() const {
  std::ostringstream ss;
  ss << "Linear (" << nIn_ << "->" << nOut_ << ")" << (bias_ ? " (with bias)" : " (without bias)");
  return ss.str();
}

}  // namespace fl
