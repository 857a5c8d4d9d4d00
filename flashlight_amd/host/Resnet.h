// ResNet building blocks and the ResNet-34 / ResNet-50 networks out of the modules of
// Modules.h, with the structure of flashlight/pkg/vision/models/Resnet.cpp:14-230
// (version 1.5: the stride sits on the 3x3 convolution of a bottleneck; no convolution
// bias, BatchNorm over axis 2 after every convolution, a 1x1 + BatchNorm projection on
// the shortcut when the shape changes).  They exercise the extension's three operators
// under the real layer mix of configs[4].
#pragma once

#include "Modules.h"

namespace fl {
namespace pkg {
namespace vision {

// BatchNorm -> ReLU and BatchNorm -> "+ shortcut" -> ReLU run as one fused operation in these
// blocks (BatchNorm::forwardRelu) unless switched off; same results to rounding, same gradients.
void setFusedBatchNormRelu(bool on);
bool fusedBatchNormRelu();

class ConvBnAct : public Sequential {
 public:
  ConvBnAct(int inC, int outC, int kw, int kh, int sx = 1, int sy = 1, bool bn = true, bool act = true);
  using Sequential::forward;
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override;

 private:
  bool bn_, act_;
};

// two 3x3 convolutions + shortcut (ResNet-18/34)
class ResNetBlock : public Container {
 public:
  ResNetBlock(int inC, int outC, int stride = 1);
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override;
  std::string prettyString() const override { return "ResNetBlock"; }
};

// 1x1 -> 3x3 (stride) -> 1x1 (x4) + shortcut (ResNet-50 and deeper)
class ResNetBottleneckBlock : public Container {
 public:
  ResNetBottleneckBlock(int inC, int planes, int stride = 1);
  std::vector<Variable> forward(const std::vector<Variable>& inputs) override;
  std::string prettyString() const override { return "ResNetBottleneckBlock"; }
};

class ResNetStage : public Sequential {
 public:
  ResNetStage(int inC, int outC, int numBlocks, int stride);
};

class ResNetBottleneckStage : public Sequential {
 public:
  ResNetBottleneckStage(int inC, int outC, int numBlocks, int stride);
};

std::shared_ptr<Sequential> resnet34();
std::shared_ptr<Sequential> resnet50();

}  // namespace vision
}  // namespace pkg
}  // namespace fl
