// nn-level wrappers over the differentiable functions of Functions.h, with the
// constructor arguments, parameter layout, initialisation and train/eval behaviour
// of the Flashlight modules they stand for (flashlight/fl/nn/modules/*.cpp), so that
// a network description written for Flashlight (Sequential of Conv2D / BatchNorm /
// ReLU / Pool2D / View / Linear / LogSoftmax, a ResNet bottleneck) reads the same
// here.  Serialization, clone() and the modules that do not touch the extension's
// operators are not provided.
#pragma once

#include <cmath>
#include <map>
#include <memory>
#include <string>
#include <unordered_set>
#include <vector>

#include "Functions.h"

namespace fl {

// ---- initialisation (flashlight/fl/nn/Init.cpp:21-48, 142-200) --------------------------
// Values are drawn on the host from one process-wide generator and copied to the device.
void setSeed(unsigned long long seed);
// 64 fresh bits of that generator: the seed of a device-side mask (dropout between rnn layers)
unsigned long long nextSeed();
Variable constant(double val, const Shape& shape, dtype type = dtype::f32, bool calcGrad = true);
Variable uniform(const Shape& shape, double min = 0, double max = 1, dtype type = dtype::f32,
                 bool calcGrad = true);
Variable kaimingUniform(const Shape& shape, int fanIn, dtype type = dtype::f32, bool calcGrad = true);
// flashlight/fl/nn/Init.cpp:19-31, 42-48, 50-68: stdv * randn + mean; kaimingNormal has stdv = sqrt(1 / fanIn);
// the Glorot pair uses stdv = sqrt(2 / (fanIn + fanOut)) (uniform: limit sqrt(3) * stdv)
Variable normal(const Shape& shape, double stdv = 1, double mean = 0, dtype type = dtype::f32, bool calcGrad = true);
Variable kaimingNormal(const Shape& shape, int fanIn, dtype type = dtype::f32, bool calcGrad = true);
Variable glorotUniform(const Shape& shape, int fanIn, int fanOut, dtype type = dtype::f32, bool calcGrad = true);
Variable glorotNormal(const Shape& shape, int fanIn, int fanOut, dtype type = dtype::f32, bool calcGrad = true);

// ---- Module (flashlight/fl/nn/modules/Module.cpp:17-112) --------------------------------
class Module {
 public:
  virtual ~Module() = default;
  std::vector<Variable> params() const { return params_; }
  int numParamTensors() const { return (int)params_.size(); }
  Variable param(int position) const;
  virtual void setParams(const Variable& var, int position);
  virtual void train();
  virtual void eval();
  bool isTrain() const { return train_; }
  void zeroGrad();
  virtual std::vector<Variable> forward(const std::vector<Variable>& inputs) = 0;
  std::vector<Variable> operator()(const std::vector<Variable>& inputs) { return forward(inputs); }
  virtual std::string prettyString() const = 0;
  // the parameters this module converts to its input's type in forward() (astype); containers
  // convert them for all their modules at once (detail::ParamCastScope)
  virtual std::vector<Variable> castParams() const { return {}; }

 protected:
  Module() = default;
  explicit Module(const std::vector<Variable>& params) : params_(params) {}
  std::vector<Variable> params_;
  bool train_ = true;
};
using ModulePtr = std::shared_ptr<Module>;

class UnaryModule : public Module {
 public:
  using Module::forward;
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override;
  virtual Variable forward(const Variable& input) = 0;
  Variable operator()(const Variable& input) { return forward(input); }

 protected:
  UnaryModule() = default;
  explicit UnaryModule(const std::vector<Variable>& params) : Module(params) {}
};

class BinaryModule : public Module {
 public:
  using Module::forward;
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override;
  virtual Variable forward(const Variable& input1, const Variable& input2) = 0;
  Variable operator()(const Variable& a, const Variable& b) { return forward(a, b); }
};

// ---- Container / Sequential (flashlight/fl/nn/modules/Container.{h,cpp}) ------------------
class Container : public Module {
 public:
  template <typename T>
  void add(std::shared_ptr<T> module) {
    if (!module) throw std::invalid_argument("can't add null Module to Container");
    for (int i = 0; i < module->numParamTensors(); ++i) {
      childParamIdx_.push_back({(int)params_.size(), (int)modules_.size(), i});
      params_.push_back(module->param(i));
    }
    modules_.emplace_back(std::move(module));
  }
  template <typename T, typename = std::enable_if_t<std::is_base_of_v<Module, std::decay_t<T>>>>
  void add(T&& module) {
    static_assert(!std::is_lvalue_reference_v<T>, "add() can only accept rvalues. Use std::move().");
    add(std::make_shared<std::decay_t<T>>(std::forward<T>(module)));
  }
  ModulePtr module(int id) const { return modules_.at(id); }
  std::vector<ModulePtr> modules() const { return modules_; }
  void train() override;
  void eval() override;
  void setParams(const Variable& var, int position) override;
  std::vector<Variable> castParams() const override;

 protected:
  struct ChildParam {
    int position, module, index;
  };
  std::vector<ModulePtr> modules_;
  std::vector<ChildParam> childParamIdx_;
};

class Sequential : public Container {
 public:
  using Module::operator();
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override;
  Variable forward(const Variable& input);
  Variable operator()(const Variable& input) { return forward(input); }
  std::string prettyString() const override;
};

// ---- layers ----------------------------------------------------------------------------
// int or PaddingMode::SAME (flashlight/fl/nn/Utils.h:40-51)
struct IntOrPadMode {
  IntOrPadMode(int v) : padVal(v) {}
  IntOrPadMode(PaddingMode m) : padVal(static_cast<int>(m)) {}
  int padVal;
};

// flashlight/fl/nn/modules/Conv2D.cpp:22-227: weight [wx, wy, nin/groups, nout] Kaiming
// uniform with fanIn = wx*wy*nin/groups, bias [1, 1, nout, 1] uniform(+-sqrt(1/fanIn))
class Conv2D : public UnaryModule {
 public:
  Conv2D(int nin, int nout, int wx, int wy, int sx = 1, int sy = 1, IntOrPadMode px = 0,
         IntOrPadMode py = 0, int dx = 1, int dy = 1, bool bias = true, int groups = 1);
  explicit Conv2D(const Variable& w, int sx = 1, int sy = 1, IntOrPadMode px = 0, IntOrPadMode py = 0,
                  int dx = 1, int dy = 1, int groups = 1);
  Conv2D(const Variable& w, const Variable& b, int sx = 1, int sy = 1, IntOrPadMode px = 0,
         IntOrPadMode py = 0, int dx = 1, int dy = 1, int groups = 1);
  using UnaryModule::forward;
  Variable forward(const Variable& input) override;
  std::string prettyString() const override;
  std::vector<Variable> castParams() const override { return params_; }

 protected:
  int nIn_, nOut_, xFilter_, yFilter_, xStride_, yStride_, xPad_, yPad_, xDilation_, yDilation_;
  bool bias_;
  int groups_;
  // the kernel-choice benchmarks of this layer's backward passes (flashlight/fl/nn/modules/Conv2D.h:206)
  std::shared_ptr<detail::ConvBenchmarks> benchmarks_ = std::make_shared<detail::ConvBenchmarks>();
};

// flashlight/fl/contrib/modules/AsymmetricConv1D.{h,cpp}: a convolution along dimension 0 whose window looks
// futurePart of its length ahead (0.5: symmetric, 0: causal, 1: only ahead): more padding, then the surplus results cut
class AsymmetricConv1D : public Conv2D {
 public:
  AsymmetricConv1D(int nin, int nout, int wx, int sx = 1, IntOrPadMode px = 0, float futurePart = 0.5f, int dx = 1,
                   bool bias = true, int groups = 1);
  using UnaryModule::forward;
  Variable forward(const Variable& input) override;
  std::string prettyString() const override;

 private:
  float futurePart_;
};

// flashlight/fl/nn/modules/Pool2D.cpp:19-52
class Pool2D : public UnaryModule {
 public:
  Pool2D(int wx, int wy, int sx = 1, int sy = 1, IntOrPadMode px = 0, IntOrPadMode py = 0,
         PoolingMode mode = PoolingMode::MAX);
  using UnaryModule::forward;
  Variable forward(const Variable& input) override;
  std::string prettyString() const override;

 private:
  int xFilter_, yFilter_, xStride_, yStride_, xPad_, yPad_;
  PoolingMode mode_;
};

// flashlight/fl/nn/modules/BatchNorm.cpp:20-128: momentum < 0 selects the cumulative
// average 1 / numBatchesTracked; eval mode normalises with the running statistics when
// they are tracked, with batch statistics otherwise
class BatchNorm : public UnaryModule {
 public:
  BatchNorm(int featAxis, int featSize, double momentum = 0.1, double eps = 1e-5, bool affine = true,
            bool trackStats = true);
  BatchNorm(const std::vector<int>& featAxis, int featSize, double momentum = 0.1, double eps = 1e-5,
            bool affine = true, bool trackStats = true);
  using UnaryModule::forward;
  Variable forward(const Variable& input) override;
  // relu(forward(input) + residual), residual optional (an empty Variable): the same
  // bookkeeping as forward(); one fused pass on the HIP extension in train mode
  Variable forwardRelu(const Variable& input, const Variable& residual = Variable());
  std::string prettyString() const override;
  Variable runningMean() const { return runningMean_; }
  Variable runningVar() const { return runningVar_; }
  int numBatchesTracked() const { return numBatchesTracked_; }

 private:
  std::vector<int> featAxis_;
  int featSize_;
  int numBatchesTracked_ = 0;
  Variable runningMean_, runningVar_;
  double momentum_, epsilon_;
  bool affine_, trackStats_;
};

// flashlight/fl/nn/modules/LayerNorm.cpp:20-160: normalises over `axis` by calling
// batchnorm over the complement axes; a complement that is not contiguous goes through
// fl::reorder as in the reference
constexpr int kLnVariableAxisSize = -1;
class LayerNorm : public UnaryModule {
 public:
  explicit LayerNorm(int axis, double eps = 1e-5, bool affine = true, int axisSize = kLnVariableAxisSize);
  explicit LayerNorm(const std::vector<int>& axis, double eps = 1e-5, bool affine = true,
                     int axisSize = kLnVariableAxisSize);
  using UnaryModule::forward;
  Variable forward(const Variable& input) override;
  std::string prettyString() const override;

 private:
  std::vector<int> axis_, axisComplement_;
  double epsilon_;
  bool affine_;
  int axisSize_;
};

// flashlight/fl/nn/modules/Linear.cpp:18-92: weight [out, in] Kaiming uniform (fanIn = in)
class Linear : public UnaryModule {
 public:
  Linear(int inputSize, int outputSize, bool bias = true);
  explicit Linear(const Variable& w);
  Linear(const Variable& w, const Variable& b);
  using UnaryModule::forward;
  Variable forward(const Variable& input) override;
  std::string prettyString() const override;
  std::vector<Variable> castParams() const override { return params_; }

 private:
  int nIn_, nOut_;
  bool bias_;
};

// flashlight/fl/nn/modules/RNN.cpp:19-170: one flat weight vector in cuDNN's order,
// uniform(+-sqrt(1/hidden)); forward takes {input[, hidden[, cell]]} and returns as many
// outputs as it got inputs
namespace detail {
int64_t getNumRnnParams(int inputSize, int hiddenSize, int numLayers, RnnMode mode, bool bidirectional);
}
class RNN : public Module {
 public:
  RNN(int inputSize, int hiddenSize, int numLayers, RnnMode mode, bool bidirectional = false,
      float dropProb = 0.0);
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override;
  Variable forward(const Variable& input) { return forward(std::vector<Variable>{input}).front(); }
  Variable operator()(const Variable& input) { return forward(input); }
  std::tuple<Variable, Variable> forward(const Variable& input, const Variable& hiddenState);
  std::tuple<Variable, Variable, Variable> forward(const Variable& input, const Variable& hiddenState,
                                                   const Variable& cellState);
  std::string prettyString() const override;
  std::vector<Variable> castParams() const override { return params_; }

 private:
  int inputSize_, hiddenSize_, numLayers_;
  RnnMode mode_;
  bool bidirectional_;
  float dropProb_;
};

class ReLU : public UnaryModule {          // Activations.cpp:58-70
 public:
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return relu(input); }
  std::string prettyString() const override { return "ReLU"; }
};

// the other element-wise modules of nn/modules/Activations.cpp
class Log : public UnaryModule {           // :32-34
 public:
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return log(input); }
  std::string prettyString() const override { return "Log"; }
};
class Tanh : public UnaryModule {          // :46-48
 public:
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return tanh(input); }
  std::string prettyString() const override { return "Tanh"; }
};
class HardTanh : public UnaryModule {      // :60-62
 public:
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return clamp(input, -1.0, 1.0); }
  std::string prettyString() const override { return "HardTanh"; }
};
class ReLU6 : public UnaryModule {         // :88-90
 public:
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return clamp(input, 0.0, 6.0); }
  std::string prettyString() const override { return "ReLU6"; }
};
class ELU : public UnaryModule {           // :132-139
 public:
  explicit ELU(double alpha = 1.0) : alpha_(alpha) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return elu(input, alpha_); }
  std::string prettyString() const override { return "ELU (" + std::to_string(alpha_) + ")"; }

 private:
  double alpha_;
};
class PReLU : public UnaryModule {         // :114-132: `size` parameters (1, or the extent of dimension 0) of value `value`
 public:
  explicit PReLU(int size = 1, double value = 0.25)
      : UnaryModule({constant(value, Shape({size, 1}), dtype::f32, true)}) {}
  explicit PReLU(const Variable& w) : UnaryModule({w}) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return prelu(input, params_[0].astype(input.type())); }
  std::string prettyString() const override { return "PReLU"; }
};
// fl::Embedding (nn/modules/Embedding.cpp:15-56): a [embeddingDim, numEmbeddings] table drawn uniformly from
// +-sqrt(1 / embeddingDim); forward = fl::embedding of s32 indices
class Embedding : public UnaryModule {
 public:
  Embedding(int embeddingDim, int numEmbeddings)
      : UnaryModule({uniform(Shape({embeddingDim, numEmbeddings}), -std::sqrt(1.0 / embeddingDim), std::sqrt(1.0 / embeddingDim),
                             dtype::f32, true)}),
        embeddingDim_(embeddingDim), numEmbeddings_(numEmbeddings) {}
  explicit Embedding(const Variable& w) : UnaryModule({w}), embeddingDim_((int)w.dim(0)), numEmbeddings_((int)w.dim(1)) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return embedding(input, params_[0]); }
  std::string prettyString() const override {
    return "Embedding (embeddings: " + std::to_string(numEmbeddings_) + ") (dim: " + std::to_string(embeddingDim_) + ")";
  }

 private:
  int embeddingDim_, numEmbeddings_;
};
class Sigmoid : public UnaryModule {       // :18-20
 public:
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return sigmoid(input); }
  std::string prettyString() const override { return "Sigmoid"; }
};
class LeakyReLU : public UnaryModule {     // :100-112
 public:
  explicit LeakyReLU(double slope = 0.0) : slope_(slope) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return leakyRelu(input, slope_); }
  std::string prettyString() const override { return "LeakyReLU (" + std::to_string(slope_) + ")"; }

 private:
  double slope_;
};
class ThresholdReLU : public UnaryModule { // :149-163
 public:
  explicit ThresholdReLU(double threshold = 1.0) : threshold_(threshold) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return thresholdRelu(input, threshold_); }
  std::string prettyString() const override { return "ThresholdReLU (" + std::to_string(threshold_) + ")"; }

 private:
  double threshold_;
};
// nn/modules/Identity.cpp:12-22: the inputs as they are
class Identity : public Module {
 public:
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override { return inputs; }
  std::string prettyString() const override { return "Identity"; }
};
class Swish : public UnaryModule {         // :190-196
 public:
  explicit Swish(double beta = 1.0) : beta_(beta) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return swish(input, beta_); }
  std::string prettyString() const override { return "Swish (" + std::to_string(beta_) + ")"; }

 private:
  double beta_;
};
class GatedLinearUnit : public UnaryModule {   // :164-168
 public:
  explicit GatedLinearUnit(int dim = 0) : dim_(dim) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return gatedlinearunit(input, dim_); }
  std::string prettyString() const override { return "GatedLinearUnit (" + std::to_string(dim_) + ")"; }

 private:
  int dim_;
};
// nn/modules/Dropout.cpp:18-24: the identity in eval mode
class Dropout : public UnaryModule {
 public:
  explicit Dropout(double ratio = 0.5) : ratio_(ratio) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return train_ ? dropout(input, ratio_) : input; }
  std::string prettyString() const override { return "Dropout (" + std::to_string(ratio_) + ")"; }

 private:
  double ratio_;
};
// nn/modules/Reorder.cpp:18-26
class Reorder : public UnaryModule {
 public:
  explicit Reorder(Shape dims) : dims_(std::move(dims)) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return reorder(input, dims_); }
  std::string prettyString() const override { return "Reorder " + dims_.toString(); }

 private:
  Shape dims_;
};

// nn/modules/Padding.cpp:14-20
class Padding : public UnaryModule {
 public:
  Padding(std::vector<std::pair<int, int>> padding, double val) : pad_(std::move(padding)), val_(val) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return padding(input, pad_, val_); }
  std::string prettyString() const override;

 private:
  std::vector<std::pair<int, int>> pad_;
  double val_;
};

// nn/modules/WeightNorm.{h,cpp}: the wrapped module's weight (parameter 0) is v * g / ||v||, the norm over all
// dimensions but `dim`; parameters {v, g} or {v, g, bias}.  Wraps a Linear or a Conv2D (one or two parameters).
class WeightNorm : public Module {
 public:
  WeightNorm(ModulePtr module, int dim);
  template <typename T, typename = std::enable_if_t<std::is_base_of_v<Module, std::decay_t<T>>>>
  WeightNorm(T&& module, int dim) : WeightNorm(ModulePtr(std::make_shared<std::decay_t<T>>(std::forward<T>(module))), dim) {}
  using Module::forward;
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override;
  void setParams(const Variable& var, int position) override;
  void train() override;
  void eval() override;
  ModulePtr module() const { return module_; }
  std::string prettyString() const override;

 private:
  void computeWeight();
  ModulePtr module_;
  int dim_;
};

// flashlight/fl/contrib/modules/TDSBlock.{h,cpp}: a time-depth separable block over [T, W, C, B]: convolution along
// time + ReLU + dropout with a shortcut, layer norm, two linear layers over W * C with a shortcut, layer norm
class TDSBlock : public Container {
 public:
  explicit TDSBlock(int channels, int kernelSize, int width, double dropout = 0, int innerLinearDim = 0,
                    int rightPadding = -1, bool lNormIncludeTime = true);
  using Module::forward;
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override;
  std::string prettyString() const override;
};

// flashlight/fl/contrib/modules/Residual.{h,cpp}: a chain of layers with shortcuts from the output of layer
// `fromLayer` (0 = the input) to the input of layer `toLayer` (number of layers + 1 = the output), optionally through a
// projection module, and a scale applied before a layer (or to the output)
class Residual : public Container {
 public:
  Residual() = default;
  void addScale(int beforeLayer, float scale);
  void addShortcut(int fromLayer, int toLayer);
  void addShortcut(int fromLayer, int toLayer, ModulePtr projection);
  template <typename T, typename = std::enable_if_t<std::is_base_of_v<Module, std::decay_t<T>>>>
  void addShortcut(int fromLayer, int toLayer, T&& projection) {
    addShortcut(fromLayer, toLayer, ModulePtr(std::make_shared<std::decay_t<T>>(std::forward<T>(projection))));
  }
  std::unordered_set<int> getProjectionsIndices() const { return projectionsIndices_; }
  using Module::forward;
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override;
  Variable forward(const Variable& input);
  std::string prettyString() const override;

 private:
  void checkShortcut(int fromLayer, int toLayer);
  Variable applyScale(const Variable& input, int layerIndex);
  std::map<int, std::map<int, int>> shortcut_;      // end -> (start -> projection module or -1)
  std::unordered_set<int> projectionsIndices_;
  std::map<int, float> scales_;
};

// nn/modules/PrecisionCast.cpp:14-30: every input cast to the target type (the gradient is cast back by astype)
class PrecisionCast : public Module {
 public:
  explicit PrecisionCast(dtype targetType) : targetType_(targetType) {}
  using Module::forward;
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override {
    std::vector<Variable> out;
    for (const auto& in : inputs) out.push_back(in.astype(targetType_));
    return out;
  }
  Variable forward(const Variable& input) { return input.astype(targetType_); }
  std::string prettyString() const override { return "PrecisionCast"; }

 private:
  dtype targetType_;
};

class LogSoftmax : public UnaryModule {    // Activations.cpp:180-192
 public:
  explicit LogSoftmax(int dim = 0) : dim_(dim) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return logSoftmax(input, dim_); }
  std::string prettyString() const override { return "LogSoftmax"; }

 private:
  int dim_;
};

class View : public UnaryModule {          // View.cpp:17-24
 public:
  explicit View(Shape dims) : dims_(std::move(dims)) {}
  using UnaryModule::forward;
  Variable forward(const Variable& input) override { return moddims(input, dims_); }
  std::string prettyString() const override { return "View " + dims_.toString(); }

 private:
  Shape dims_;
};

// flashlight/fl/nn/modules/Loss.cpp (CategoricalCrossEntropy)
class CategoricalCrossEntropy : public BinaryModule {
 public:
  explicit CategoricalCrossEntropy(ReduceMode reduction = ReduceMode::MEAN, int ignoreIndex = -1)
      : reduction_(reduction), ignoreIndex_(ignoreIndex) {}
  using BinaryModule::forward;
  Variable forward(const Variable& inputs, const Variable& targets) override {
    return categoricalCrossEntropy(inputs, targets, reduction_, ignoreIndex_);
  }
  std::string prettyString() const override { return "CategoricalCrossEntropy"; }

 private:
  ReduceMode reduction_;
  int ignoreIndex_;
};

}  // namespace fl
