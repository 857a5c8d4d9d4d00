#include "Resnet.h"

namespace fl {
namespace pkg {
namespace vision {

namespace {
const auto kSame = PaddingMode::SAME;

std::shared_ptr<Conv2D> conv(int inC, int outC, int k, int stride) {
  return std::make_shared<Conv2D>(inC, outC, k, k, stride, stride, kSame, kSame, 1, 1, /* bias */ false);
}

// projection shortcut (Resnet.cpp:57-62, 83-88)
std::shared_ptr<Sequential> projection(int inC, int outC, int stride) {
  auto s = std::make_shared<Sequential>();
  s->add(conv(inC, outC, 1, stride));
  s->add(std::make_shared<BatchNorm>(2, outC));
  return s;
}

bool g_fuse = true;

BatchNorm* asBatchNorm(const std::shared_ptr<Module>& m) { return dynamic_cast<BatchNorm*>(m.get()); }

// main path through modules [0, last) in groups of (convolution, BatchNorm, ReLU), plus the
// shortcut, then the final ReLU (Resnet.cpp:95-140)
std::vector<Variable> residual(const Container& c, int mainModules, const std::vector<Variable>& inputs) {
  std::vector<Variable> out = inputs;
  const std::vector<Variable> shortcut =
      (int)c.modules().size() > mainModules ? c.module(mainModules)->forward(inputs) : inputs;
  if (!g_fuse) {
    for (int i = 0; i + 1 < mainModules; ++i) out = c.module(i)->forward(out);
    return c.module(mainModules - 1)->forward({out[0] + shortcut[0]});
  }
  for (int i = 0; i < mainModules; i += 3) {
    out = c.module(i)->forward(out);
    BatchNorm* bn = asBatchNorm(c.module(i + 1));
    const bool last = i + 3 >= mainModules;
    if (bn) {
      out = {bn->forwardRelu(out[0], last ? shortcut[0] : Variable())};
    } else {
      out = c.module(i + 1)->forward(out);
      out = c.module(i + 2)->forward(last ? std::vector<Variable>{out[0] + shortcut[0]} : out);
    }
  }
  return out;
}
}  // namespace

void setFusedBatchNormRelu(bool on) { g_fuse = on; }
bool fusedBatchNormRelu() { return g_fuse; }

std::vector<Variable> ConvBnAct::forward(const std::vector<Variable>& inputs) {
  if (!(g_fuse && bn_ && act_)) return Sequential::forward(inputs);
  std::vector<Variable> out = module(0)->forward(inputs);
  return {asBatchNorm(module(1))->forwardRelu(out[0])};
}

ConvBnAct::ConvBnAct(int inC, int outC, int kw, int kh, int sx, int sy, bool bn, bool act) : bn_(bn), act_(act) {
  add(std::make_shared<Conv2D>(inC, outC, kw, kh, sx, sy, kSame, kSame, 1, 1, /* bias */ !bn));
  if (bn) add(std::make_shared<BatchNorm>(2, outC));
  if (act) add(std::make_shared<ReLU>());
}

ResNetBlock::ResNetBlock(int inC, int outC, int stride) {
  add(conv(inC, outC, 3, stride));
  add(std::make_shared<BatchNorm>(2, outC));
  add(std::make_shared<ReLU>());
  add(conv(outC, outC, 3, 1));
  add(std::make_shared<BatchNorm>(2, outC));
  add(std::make_shared<ReLU>());
  if (inC != outC || stride > 1) add(projection(inC, outC, stride));
}

std::vector<Variable> ResNetBlock::forward(const std::vector<Variable>& inputs) {
  return residual(*this, 6, inputs);
}

ResNetBottleneckBlock::ResNetBottleneckBlock(int inC, int planes, int stride) {
  const int expansion = 4;
  add(conv(inC, planes, 1, 1));
  add(std::make_shared<BatchNorm>(2, planes));
  add(std::make_shared<ReLU>());
  add(conv(planes, planes, 3, stride));
  add(std::make_shared<BatchNorm>(2, planes));
  add(std::make_shared<ReLU>());
  add(conv(planes, planes * expansion, 1, 1));
  add(std::make_shared<BatchNorm>(2, planes * expansion));
  add(std::make_shared<ReLU>());
  if (inC != planes * expansion || stride > 1) add(projection(inC, planes * expansion, stride));
}

std::vector<Variable> ResNetBottleneckBlock::forward(const std::vector<Variable>& inputs) {
  return residual(*this, 9, inputs);
}

ResNetStage::ResNetStage(int inC, int outC, int numBlocks, int stride) {
  add(std::make_shared<ResNetBlock>(inC, outC, stride));
  for (int i = 1; i < numBlocks; ++i) add(std::make_shared<ResNetBlock>(outC, outC));
}

ResNetBottleneckStage::ResNetBottleneckStage(int inC, int outC, int numBlocks, int stride) {
  add(std::make_shared<ResNetBottleneckBlock>(inC, outC, stride));
  for (int i = 1; i < numBlocks; ++i) add(std::make_shared<ResNetBottleneckBlock>(outC * 4, outC));
}

namespace {
std::shared_ptr<Sequential> stem() {
  auto model = std::make_shared<Sequential>();
  model->add(std::make_shared<ConvBnAct>(3, 64, 7, 7, 2, 2));                        // 224 -> 112
  model->add(std::make_shared<Pool2D>(3, 3, 2, 2, kSame, kSame, PoolingMode::MAX));  // 112 -> 56
  return model;
}
void head(Sequential& model, int features) {
  model.add(std::make_shared<Pool2D>(7, 7, 1, 1, 0, 0, PoolingMode::AVG_EXCLUDE_PADDING));
  model.add(std::make_shared<View>(Shape({features, -1})));
  model.add(std::make_shared<Linear>(features, 1000));
}
}  // namespace

std::shared_ptr<Sequential> resnet34() {
  auto model = stem();
  model->add(std::make_shared<ResNetStage>(64, 64, 3, 1));
  model->add(std::make_shared<ResNetStage>(64, 128, 4, 2));
  model->add(std::make_shared<ResNetStage>(128, 256, 6, 2));
  model->add(std::make_shared<ResNetStage>(256, 512, 3, 2));
  head(*model, 512);
  return model;
}

std::shared_ptr<Sequential> resnet50() {
  auto model = stem();
  model->add(std::make_shared<ResNetBottleneckStage>(64, 64, 3, 1));
  model->add(std::make_shared<ResNetBottleneckStage>(64 * 4, 128, 4, 2));
  model->add(std::make_shared<ResNetBottleneckStage>(128 * 4, 256, 6, 2));
  model->add(std::make_shared<ResNetBottleneckStage>(256 * 4, 512, 3, 2));
  head(*model, 512 * 4);
  return model;
}

}  // namespace vision
}  // namespace pkg
}  // namespace fl
