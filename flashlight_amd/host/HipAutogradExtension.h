// AutogradExtension for MI355X: every op lowers to one C ABI call of libflhip on
// device-resident tensors.  Peer of OneDnnAutogradExtension / CudnnAutogradExtension
// (flashlight/fl/autograd/tensor/backend/{onednn,cudnn}).
#pragma once

#include "AutogradExtension.h"

namespace fl {

class HipAutogradExtension : public AutogradExtension {
 public:
  // refuses to run on a libflhip whose descriptor layouts differ from the header this class was compiled with
  HipAutogradExtension();
  // One benchmark of a backward pass of one convolution: its options are "the default rule" and every kernel
  // family of libflhip's backward passes (flhip_conv2d_plan_count), each timed kPlanBenchCount times on the first
  // calls made in benchmark mode; the fastest then runs every later call with the same geometry (a call with
  // another geometry starts the timings again).  The cuDNN peer offers its three kernel modes the same way
  // (cudnn/CudnnAutogradExtension.cpp:17-25).
  std::shared_ptr<DynamicBenchmark> createBenchmarkOptions() override;
  static constexpr int kPlanBenchCount = 3;
  // f32, f16 and the private bf16 tag (the 16-bit types are storage types: sums are fp32).  The oneDNN
  // extension supports everything but f16 (onednn/OneDnnAutogradExtension.cpp:12-16), the cuDNN one f16/f32/f64.
  bool isDataTypeSupported(const dtype& type) const override;

  Tensor conv2d(const Tensor& input, const Tensor& weights, const Tensor& bias, const int sx,
                const int sy, const int px, const int py, const int dx, const int dy,
                const int groups, std::shared_ptr<detail::AutogradPayload> payload) override;
  Tensor pool2d(const Tensor& input, const int wx, const int wy, const int sx, const int sy,
                const int px, const int py, const PoolingMode mode,
                std::shared_ptr<detail::AutogradPayload> payload) override;
  Tensor batchnorm(Tensor& saveMean, Tensor& saveVar, const Tensor& input, const Tensor& weight,
                   const Tensor& bias, Tensor& runningMean, Tensor& runningVar,
                   const std::vector<int>& axes, const bool train, const double momentum,
                   const double epsilon, std::shared_ptr<detail::AutogradPayload> payload) override;
  std::tuple<Tensor, Tensor, Tensor> rnn(const Tensor&, const Tensor&, const Tensor&,
                                         const Tensor&, const int, const int, const RnnMode,
                                         const bool, const float,
                                         std::shared_ptr<detail::AutogradPayload>) override;

  Tensor conv2dBackwardData(const Tensor& gradOutput, const Tensor& input, const Tensor& weight,
                            const int sx, const int sy, const int px, const int py, const int dx,
                            const int dy, const int groups,
                            std::shared_ptr<DynamicBenchmark> dataGradBenchmark,
                            std::shared_ptr<detail::AutogradPayload> payload) override;
  std::pair<Tensor, Tensor> conv2dBackwardFilterBias(
      const Tensor& gradOutput, const Tensor& input, const Tensor& weights, const Tensor& bias,
      const int sx, const int sy, const int px, const int py, const int dx, const int dy,
      const int groups, std::shared_ptr<DynamicBenchmark> filterBench,
      std::shared_ptr<DynamicBenchmark> biasBench,
      std::shared_ptr<detail::AutogradPayload> autogradPayload) override;
  Tensor pool2dBackward(const Tensor& gradOutput, const Tensor& input, const Tensor& poolOutput,
                        const int wx, const int wy, const int sx, const int sy, const int px,
                        const int py, const PoolingMode mode,
                        std::shared_ptr<detail::AutogradPayload> payload) override;
  std::tuple<Tensor, Tensor, Tensor> batchnormBackward(
      const Tensor& gradOutput, const Tensor& saveMean, const Tensor& saveVar, const Tensor& input,
      const Tensor& weight, const std::vector<int>& axes, const bool train, const float epsilon,
      std::shared_ptr<detail::AutogradPayload> payload) override;
  std::tuple<Tensor, Tensor, Tensor, Tensor> rnnBackward(
      const Tensor&, const Tensor&, const Tensor&, const Tensor&,
      const std::shared_ptr<detail::RNNGradData>, const Tensor&, const int, const int,
      const RnnMode, const bool, const float, std::shared_ptr<detail::AutogradPayload>) override;

  // Not part of fl::AutogradExtension: batch norm (train mode, feature axes not starting at
  // dimension 0) fused with the residual add and the ReLU that follow it in a ResNet block,
  // output = relu(batchnorm(input) + residual) (residual may be empty), and its backward,
  // which returns (gradInput, gradWeight, gradBias, gradResidual); gradResidual is only
  // produced when wantResidualGrad.  fl::detail::batchnormRelu reaches them when the tensor's
  // extension is this class and composes the three reference operators otherwise.
  Tensor batchnormRelu(Tensor& saveMean, Tensor& saveVar, const Tensor& input, const Tensor& weight,
                       const Tensor& bias, Tensor& runningMean, Tensor& runningVar,
                       const std::vector<int>& axes, const double momentum, const double epsilon,
                       const Tensor& residual, std::shared_ptr<detail::AutogradPayload> payload);
  // addend + conv2dBackwardData(...): the closure's backward-data pass and the addGrad behind it
  // in one pass over the result (flhip_conv2d_bwd_data_add)
  Tensor conv2dBackwardDataAdd(const Tensor& gradOutput, const Tensor& input, const Tensor& weights,
                               const Tensor& addend, const int sx, const int sy, const int px, const int py,
                               const int dx, const int dy, const int groups);
  std::tuple<Tensor, Tensor, Tensor, Tensor> batchnormReluBackward(
      const Tensor& gradOutput, const Tensor& output, const Tensor& saveMean, const Tensor& saveVar,
      const Tensor& input, const Tensor& weight, const std::vector<int>& axes, const bool wantResidualGrad,
      std::shared_ptr<detail::AutogradPayload> payload);

 private:
  Tensor workspace(size_t bytes);   // grown on demand, reused across calls
  Tensor ws_;
};

}  // namespace fl
