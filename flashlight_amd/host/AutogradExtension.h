// The operator interface of the boundary: fl::AutogradExtension with the virtual
// signatures of flashlight/fl/autograd/tensor/AutogradExtension.h:46-180, and the
// registration mechanism of flashlight/fl/tensor/TensorExtension.{h,cpp}.
#pragma once

#include <functional>
#include <memory>
#include <tuple>
#include <utility>
#include <vector>

#include "HipTensor.h"

namespace fl {

namespace detail {
// gradients of the three rnn outputs, filled by the closures of the outputs that were
// differentiated (flashlight/fl/autograd/tensor/AutogradOps.h:356-360)
struct RNNGradData {
  Tensor dy, dhy, dcy;
};
// Opaque forward -> backward state (AutogradExtension.h:26-42).  The caller
// creates the payload only when some input needs a gradient
// (flashlight/fl/autograd/Functions.h:84-89); the forward op fills `data`.
struct AutogradPayloadData {
  virtual ~AutogradPayloadData() = default;
};
struct AutogradPayload {
  std::shared_ptr<AutogradPayloadData> data;
};
}  // namespace detail

class AutogradExtension {
 public:
  virtual ~AutogradExtension() = default;
  static constexpr TensorExtensionType extensionType = TensorExtensionType::Autograd;

  virtual bool isDataTypeSupported(const dtype& type) const = 0;
  virtual std::shared_ptr<DynamicBenchmark> createBenchmarkOptions() { return nullptr; }

  /**************************** Forward ****************************/
  virtual Tensor conv2d(const Tensor& input, const Tensor& weights, const Tensor& bias,
                        const int sx, const int sy, const int px, const int py, const int dx,
                        const int dy, const int groups,
                        std::shared_ptr<detail::AutogradPayload> payload) = 0;
  virtual Tensor pool2d(const Tensor& input, const int wx, const int wy, const int sx,
                        const int sy, const int px, const int py, const PoolingMode mode,
                        std::shared_ptr<detail::AutogradPayload> payload) = 0;
  virtual Tensor batchnorm(Tensor& saveMean, Tensor& saveVar, const Tensor& input,
                           const Tensor& weight, const Tensor& bias, Tensor& runningMean,
                           Tensor& runningVar, const std::vector<int>& axes, const bool train,
                           const double momentum, const double epsilon,
                           std::shared_ptr<detail::AutogradPayload> payload) = 0;
  virtual std::tuple<Tensor, Tensor, Tensor> rnn(
      const Tensor& input, const Tensor& hiddenState, const Tensor& cellState,
      const Tensor& weights, const int hiddenSize, const int numLayers, const RnnMode mode,
      const bool bidirectional, const float dropout,
      std::shared_ptr<detail::AutogradPayload> payload) = 0;

  /**************************** Backward ****************************/
  virtual Tensor conv2dBackwardData(const Tensor& gradOutput, const Tensor& input,
                                    const Tensor& weight, const int sx, const int sy,
                                    const int px, const int py, const int dx, const int dy,
                                    const int groups,
                                    std::shared_ptr<DynamicBenchmark> dataGradBenchmark,
                                    std::shared_ptr<detail::AutogradPayload> payload) = 0;
  virtual std::pair<Tensor, Tensor> conv2dBackwardFilterBias(
      const Tensor& gradOutput, const Tensor& input, const Tensor& weights, const Tensor& bias,
      const int sx, const int sy, const int px, const int py, const int dx, const int dy,
      const int groups, std::shared_ptr<DynamicBenchmark> filterBench,
      std::shared_ptr<DynamicBenchmark> biasBench,
      std::shared_ptr<detail::AutogradPayload> autogradPayload) = 0;
  virtual Tensor pool2dBackward(const Tensor& gradOutput, const Tensor& input,
                                const Tensor& poolOutput, const int wx, const int wy,
                                const int sx, const int sy, const int px, const int py,
                                const PoolingMode mode,
                                std::shared_ptr<detail::AutogradPayload> payload) = 0;
  virtual std::tuple<Tensor, Tensor, Tensor> batchnormBackward(
      const Tensor& gradOutput, const Tensor& saveMean, const Tensor& saveVar,
      const Tensor& input, const Tensor& weight, const std::vector<int>& axes, const bool train,
      const float epsilon, std::shared_ptr<detail::AutogradPayload> payload) = 0;
  virtual std::tuple<Tensor, Tensor, Tensor, Tensor> rnnBackward(
      const Tensor& input, const Tensor& hiddenState, const Tensor& cellState,
      const Tensor& weights, const std::shared_ptr<detail::RNNGradData> gradData,
      const Tensor& output, const int numLayers, const int hiddenSize, const RnnMode mode,
      const bool bidirectional, const float dropProb,
      std::shared_ptr<detail::AutogradPayload> payload) = 0;
};

// Registry keyed by (backend, extension type); the first registration wins and
// later ones are ignored (flashlight/fl/tensor/TensorExtension.cpp:14-30).  One
// extension instance per backend, created lazily on first use
// (flashlight/fl/tensor/TensorBackend.h:282-300).
namespace detail {
using AutogradExtensionFactory = std::function<std::unique_ptr<AutogradExtension>()>;
bool registerAutogradExtension(TensorBackendType backend, AutogradExtensionFactory f);
}  // namespace detail

// input.backend().getExtension<AutogradExtension>() of the reference.
AutogradExtension& getAutogradExtension(TensorBackendType backend);

#define FL_REGISTER_AUTOGRAD_EXTENSION(TYPE, BACKEND)                                   \
  static const bool flRegistered##TYPE##BACKEND = ::fl::detail::registerAutogradExtension( \
      ::fl::TensorBackendType::BACKEND, [] { return std::unique_ptr<::fl::AutogradExtension>(new TYPE()); })

}  // namespace fl
