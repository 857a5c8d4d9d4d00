// The caller side of the boundary: a minimal autograd Variable and the three
// differentiable functions whose closures drive the extension, with the control
// flow of flashlight/fl/autograd/Functions.cpp:1327-1565 (dtype checks, payload
// creation, which backward op runs when) and the reverse-topological backward of
// flashlight/fl/autograd/Variable.cpp:235-294; plus the few functions a network of
// those layers needs to run a training step on the device (relu, linear, moddims,
// logSoftmax, categoricalCrossEntropy).  Only what is needed to exercise the
// extension the way Flashlight does is provided.
#pragma once

#include <functional>
#include <memory>
#include <tuple>
#include <utility>
#include <vector>

#include "DynamicBenchmark.h"
#include "AutogradExtension.h"

namespace fl {

class Variable {
 public:
  using GradFunc = std::function<void(std::vector<Variable>& inputs, const Variable& gradOutput)>;

  Variable() : data_(std::make_shared<Tensor>()), grad_(std::make_shared<SharedGrad>()) {}
  Variable(Tensor data, bool calcGrad);
  Variable(Tensor data, std::vector<Variable> inputs, GradFunc gradFunc);

  Tensor& tensor() const { return *data_; }
  const Shape& shape() const { return data_->shape(); }
  dtype type() const { return data_->type(); }
  bool isEmpty() const { return data_->isEmpty(); }
  int ndim() const { return data_->ndim(); }
  Dim dim(int i) const { return data_->dim(i); }
  Dim elements() const { return data_->elements(); }
  bool isCalcGrad() const { return grad_->calcGrad; }
  // flashlight/fl/autograd/Variable.cpp:155-163: switching off also drops the graph
  void setCalcGrad(bool calcGrad);
  // differentiable cast (Variable.cpp:100-108); among f32, bf16 and f16 here
  Variable astype(dtype type) const;
  // the cast node of this variable around a conversion that was made elsewhere (one of many in
  // one launch): same graph node as astype() builds
  Variable castNode(const Tensor& converted) const;
  // identity of the variable's shared state (copies of a Variable share it)
  const void* id() const { return grad_.get(); }
  bool isGradAvailable() const { return grad_->grad != nullptr; }
  Variable& grad() const;
  void addGrad(const Variable& childGrad);
  // Adds a gradient that an operation produced in a wider type than this Variable (the fp32
  // filter / bias gradients of a convolution over bf16 storage).  When this Variable is a cast
  // of one that has the gradient's type (astype of an fp32 master parameter), the gradient
  // goes to that one as it is: the reference's path, astype to this type here and back in the
  // cast's own gradient function (Functions.cpp:1391-1410, Variable.cpp:100-108), rounds it to
  // the narrow type for nothing and costs two conversion kernels per parameter.  Otherwise
  // the same as addGrad(astype).
  void addGradWide(const Tensor& grad);
  void zeroGrad() { grad_->grad.reset(); }
  // the gradient accumulated so far is replaced by `sum` (an operation that added its own
  // contribution to it in the pass that produced it)
  void replaceGrad(const Tensor& sum) { grad_->grad.reset(new Variable(sum, false)); }
  void backward(const Variable& grad, bool retainGraph = false);

 private:
  struct SharedGrad {
    bool calcGrad = false;
    bool isCast = false;   // result of astype(): inputs[0] is the source
    std::vector<Variable> inputs;
    std::unique_ptr<Variable> grad;
    GradFunc gradFunc;
  };
  std::vector<Variable> build() const;   // nodes in topological order
  std::shared_ptr<Tensor> data_;
  std::shared_ptr<SharedGrad> grad_;
};

// fl::derivePadding (flashlight/fl/nn/Utils.cpp:87-100); pad == -1 is SAME
int derivePadding(int inSz, int filterSz, int stride, int pad, int dilation);

// `benchmarks` (flashlight/fl/autograd/Functions.h: the last argument of both forms): where the backward passes keep
// their kernel-choice benchmarks between calls; created on the first backward pass made in benchmark mode.
Variable conv2d(const Variable& input, const Variable& weights, const Variable& bias, int sx = 1,
                int sy = 1, int px = 0, int py = 0, int dx = 1, int dy = 1, int groups = 1,
                std::shared_ptr<detail::ConvBenchmarks> benchmarks = nullptr);
Variable conv2d(const Variable& input, const Variable& weights, int sx = 1, int sy = 1,
                int px = 0, int py = 0, int dx = 1, int dy = 1, int groups = 1,
                std::shared_ptr<detail::ConvBenchmarks> benchmarks = nullptr);
Variable pool2d(const Variable& input, int wx, int wy, int sx = 1, int sy = 1, int px = 0,
                int py = 0, PoolingMode mode = PoolingMode::MAX);
Variable batchnorm(const Variable& input, const Variable& weight, const Variable& bias,
                   Variable& runningMean, Variable& runningVar, const std::vector<int>& axes,
                   bool train, double momentum, double epsilon);

// fl::rnn (Functions.cpp:1606-1706): input [input, batch, seq], states [hidden, batch,
// layers*dirs] (empty = zeros), weights flat in cuDNN's order -> (output, hidden, cell)
std::tuple<Variable, Variable, Variable> rnn(const Variable& input, const Variable& hiddenState,
                                             const Variable& cellState, const Variable& weights,
                                             int hiddenSize, int numLayers, RnnMode mode,
                                             bool bidirectional, float dropProb);

// flashlight/fl/common/Defines.h:83-87
enum class ReduceMode { NONE = 0, MEAN = 1, SUM = 2 };

// input + other, same shapes (the residual add; Functions.cpp:111-121)
Variable add(const Variable& lhs, const Variable& rhs);
inline Variable operator+(const Variable& lhs, const Variable& rhs) { return add(lhs, rhs); }
namespace detail {
// While a ParamCastScope is alive, Variable::astype(to) of the variables it was given returns the
// cast node the scope made for it: all of them converted in one launch (Tensor::astypeMany)
// instead of one launch per module and step.  Nested scopes do nothing; the outermost one owns
// the nodes and drops them when it ends (the graph keeps the ones it uses).
class ParamCastScope {
 public:
  ParamCastScope(const std::vector<Variable>& params, dtype to);
  ~ParamCastScope();
  ParamCastScope(const ParamCastScope&) = delete;
  ParamCastScope& operator=(const ParamCastScope&) = delete;

 private:
  bool owner_ = false;
};
// Whether the backward-data pass of fl::conv2d adds the gradient its input already holds in the
// pass that writes its result (HipAutogradExtension::conv2dBackwardDataAdd) instead of leaving
// the sum to Variable::addGrad.  The values are the same bit for bit.  Default: on.
void setFusedGradAdd(bool on);
bool fusedGradAdd();
// relu(batchnorm(input, ...) + residual) in train mode, residual optional (an empty Variable):
// the tail of a ResNet block (flashlight/pkg/vision/models/Resnet.cpp:95-140).  On the HIP
// extension with feature axes that do not start at dimension 0 this is one fused pass forward
// and one backward; otherwise the three reference functions are composed.  Same gradients
// either way.
Variable batchnormRelu(const Variable& input, const Variable& weight, const Variable& bias,
                       Variable& runningMean, Variable& runningVar, const std::vector<int>& axes,
                       double momentum, double epsilon, const Variable& residual);
// tileAs(weight, input) * input + tileAs(bias, input) on the [outer][mid][inner] view of
// the input, one parameter element per mid index or a single one (scalar): the affine
// part of LayerNorm (flashlight/fl/nn/modules/LayerNorm.cpp:110-128)
Variable affine(const Variable& input, const Variable& weight, const Variable& bias, Dim outer,
                Dim mid, Dim inner, bool scalar);
}  // namespace detail

// fl::relu = max(input, 0) (Functions.cpp:329-338, 1787-1789)
Variable relu(const Variable& input);
// fl::moddims / View: same data, new shape; one dimension may be -1 (Functions.cpp:790-829)
// The other element-wise activations (flashlight/fl/autograd/Functions.cpp:403-411 log, :454-463 tanh, :465-475 clamp,
// :488-496 sigmoid, :498-500 swish; nn/modules/Activations.cpp:136-139 elu).  clamp passes the gradient where
// lo < result < hi.
Variable elu(const Variable& input, double alpha = 1.0);
Variable clamp(const Variable& input, double lo, double hi);
Variable tanh(const Variable& input);
Variable log(const Variable& input);
Variable sigmoid(const Variable& input);
Variable swish(const Variable& input, double beta);
// LeakyReLU's max(input, slope * input) and ThresholdReLU's input * (input >= threshold) as one operator each
// (nn/modules/Activations.cpp:102-104, 151-154; the first with fl::max's gradient mask, Functions.cpp:315-327)
Variable leakyRelu(const Variable& input, double slope);
Variable thresholdRelu(const Variable& input, double threshold);
// a Variable times a number (the reference's operator*(Variable, double))
Variable scale(const Variable& input, double factor);
inline Variable operator*(const Variable& lhs, double rhs) { return scale(lhs, rhs); }
inline Variable operator*(double lhs, const Variable& rhs) { return scale(rhs, lhs); }
// fl::PReLU's forward (nn/modules/Activations.cpp:121-124) as one operator: input where input >= 0, input * weight
// elsewhere, the weight tiled along dimension 0 (one element, or one per index of dimension 0).  Same dtype for both.
Variable prelu(const Variable& input, const Variable& weight);
// fl::embedding (Functions.cpp:1707-1749): input = s32 indices of at most 3 dims, embeddings [dim, tokens] ->
// [dim, input dims...]; the gradient goes to the embeddings only
Variable embedding(const Variable& input, const Variable& embeddings);
// fl::gatedlinearunit (Functions.cpp:1567-1610): first half of dimension `dim` times the sigmoid of the second half
Variable gatedlinearunit(const Variable& input, int dim);
// fl::dropout (Functions.cpp:1777-1785): input * mask / (1 - p); p <= 0 returns the input.  The mask is a
// counter-based function of a seed drawn from the process-wide generator (fl::setSeed), regenerated by the
// backward pass.
Variable dropout(const Variable& input, double p);
// The weight of fl::WeightNorm (nn/modules/WeightNorm.cpp:45-66): v * tileAs(g / norm(v over all dimensions but
// `dim`), v); dim is 0 or the last dimension of v (the reference: 0 or 3 of four).  g has one element per index of
// `dim`.  rowNorm gives those norms with the kept-dimensions shape (the initial g, :68-72).
Variable weightNorm(const Variable& v, const Variable& g, int dim);
Tensor rowNorm(const Tensor& v, int dim);
// fl::padding (Functions.cpp:1751-1775): pad[i] = (before, after) for dimension i, filled with val
Variable padding(const Variable& input, const std::vector<std::pair<int, int>>& pad, double val);
// input(range(start, start + size)) along dimension dim, as the reference's indexing of a Variable with a range: the
// gradient is the incoming one inside zeros
Variable narrow(const Variable& input, int dim, long long start, long long size);
Variable moddims(const Variable& input, const Shape& dims);
// fl::reorder (Functions.cpp:1010-1042): dimension k of the result is dimension dims[k] of the
// input; the gradient is reordered back with the inverse permutation
Variable reorder(const Variable& input, const Shape& dims);
// fl::linear (Functions.cpp:1255-1309): weight [out, in], input [in, ...], bias [out] or empty
Variable linear(const Variable& input, const Variable& weight, const Variable& bias);
Variable linear(const Variable& input, const Variable& weight);
// fl::logSoftmax over dimension 0 (Functions.cpp:1044-1070; other dimensions throw here)
Variable logSoftmax(const Variable& input, int dim);
// fl::categoricalCrossEntropy (Functions.cpp:1078-1154): input [C, X...] log-probabilities,
// targets [X...] of type s32
Variable categoricalCrossEntropy(const Variable& input, const Variable& targets,
                                 ReduceMode reduction = ReduceMode::MEAN, int ignoreIndex = -1);

}  // namespace fl
