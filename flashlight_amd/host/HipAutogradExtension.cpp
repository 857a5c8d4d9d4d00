#include "HipAutogradExtension.h"
#include "DynamicBenchmark.h"
#include "OpObserver.h"

#include <algorithm>
#include <cstring>
#include <map>
#include <mutex>
#include <string>

#include "flhip.h"

namespace fl {

// ---- registry ---------------------------------------------------------------
namespace detail {
namespace {
struct Registry {
  std::mutex m;
  std::map<TensorBackendType, AutogradExtensionFactory> factories;
  std::map<TensorBackendType, std::unique_ptr<AutogradExtension>> instances;
};
Registry& registry() {
  // never destroyed: extension instances own device tensors (their workspace), and a
  // process may unload the HIP runtime before its own static destructors run
  static Registry* r = new Registry;
  return *r;
}
}  // namespace

bool registerAutogradExtension(TensorBackendType backend, AutogradExtensionFactory f) {
  Registry& r = registry();
  std::lock_guard<std::mutex> lock(r.m);
  // try_emplace semantics: the first registration for a backend stays
  return r.factories.emplace(backend, std::move(f)).second;
}
}  // namespace detail

AutogradExtension& getAutogradExtension(TensorBackendType backend) {
  auto& r = detail::registry();
  std::lock_guard<std::mutex> lock(r.m);
  auto it = r.instances.find(backend);
  if (it == r.instances.end()) {
    auto f = r.factories.find(backend);
    if (f == r.factories.end())
      throw std::invalid_argument("no AutogradExtension registered for this tensor backend");
    it = r.instances.emplace(backend, f->second()).first;
  }
  return *it->second;
}

// registers next to the cuDNN / oneDNN extensions of
// flashlight/fl/autograd/tensor/AutogradExtensionBackends.h:28-42
FL_REGISTER_AUTOGRAD_EXTENSION(HipAutogradExtension, Hip);

// ---- helpers ----------------------------------------------------------------
namespace {

// status of the C ABI -> the exception kinds of the reference boundary
// (flashlight/fl/autograd/tensor/backend/cudnn/CudnnUtils.cpp:88-99)
void check(int rc) {
  if (rc == FLHIP_OK) return;
  if (rc == FLHIP_INVALID_ARGUMENT) throw std::invalid_argument(flhip_last_error());
  throw std::runtime_error(flhip_last_error());
}

int dtypeTag(dtype t, const char* op) {
  if (t == dtype::f32) return FLHIP_F32;
  if (t == dtype::bf16) return FLHIP_BF16;
  if (t == dtype::f16) return FLHIP_F16;
  throw std::runtime_error(std::string(op) + ": data type not supported by the HIP autograd extension");
}

// fp32 view of a small parameter vector (bias, gamma, beta, statistics)
Tensor asF32(const Tensor& t) { return (t.isEmpty() || t.type() == dtype::f32) ? t : t.astype(dtype::f32); }

struct HipPool2DPayload : detail::AutogradPayloadData {
  Tensor argmax;   // one byte per output: first maximum, window-relative index
};
struct HipConv2DPayload : detail::AutogradPayloadData {
  Tensor gathered;   // the forward pass's workspace of a strided bf16 layer: it starts with the gathered input,
                     // which conv2dBackwardFilterBias takes in place of gathering again
};
struct HipBatchNormPayload : detail::AutogradPayloadData {
  Tensor saveMean, saveInvStd;   // fp32 per feature
  Tensor reluMask;               // batchnormRelu: one byte per 4 elements of the result, bit e = (y[4i+e] > 0)
};

flhip_conv_desc convDesc(const Shape& in, const Tensor& weights, int sx, int sy, int px, int py,
                         int dx, int dy, int groups, int tag, const char* op) {
  if (in.ndim() != 4 || weights.ndim() != 4)
    throw std::invalid_argument(std::string(op) + ": input and weights must have 4 dimensions");
  flhip_conv_desc d{};
  d.W = (int)in.dim(0); d.H = (int)in.dim(1); d.C = (int)in.dim(2); d.N = (int)in.dim(3);
  d.KW = (int)weights.dim(0); d.KH = (int)weights.dim(1); d.K = (int)weights.dim(3);
  d.sx = sx; d.sy = sy; d.px = px; d.py = py; d.dil_x = dx; d.dil_y = dy;
  d.groups = groups; d.dtype = tag;
  if (groups <= 0 || weights.dim(2) * groups != in.dim(2))
    throw std::invalid_argument(std::string(op) + ": weights do not match the input channels");
  return d;
}

// (outer, C, inner) of the view of onednn/BatchNorm.cpp:40-71 with the axis
// check of :124-130
flhip_bn_desc bnDesc(const Tensor& input, const std::vector<int>& axes, int tag) {
  if (axes.empty()) throw std::invalid_argument("batchnorm: no feature axes");
  const int maxAxis = *std::max_element(axes.begin(), axes.end());
  const int minAxis = *std::min_element(axes.begin(), axes.end());
  if ((int)axes.size() != maxAxis - minAxis + 1 || minAxis < 0 || maxAxis >= input.ndim())
    throw std::invalid_argument("axis array should be continuous");
  long long nfeat = 1;
  for (int ax : axes) nfeat *= input.dim(ax);
  flhip_bn_desc d{};
  d.C = nfeat;
  d.dtype = tag;
  if (minAxis == 0) {
    d.inner = 1;
    d.outer = input.elements() / nfeat;
  } else {
    long long batch = 1;
    for (int i = maxAxis + 1; i < input.ndim(); ++i) batch *= input.dim(i);
    d.outer = batch;
    d.inner = input.elements() / (nfeat * batch);
  }
  return d;
}

}  // namespace

HipAutogradExtension::HipAutogradExtension() {
  if (flhip_version() / 100 != FLHIP_VERSION / 100)
    throw std::runtime_error("HipAutogradExtension: libflhip version " + std::to_string(flhip_version()) +
                             " does not match the header it was compiled with (" + std::to_string(FLHIP_VERSION) + ")");
}

// ---- plans of the backward passes -------------------------------------------------------------
namespace {
// option -1 = the default rule, 0 .. = the kernel families; remembers the geometry its timings belong to
struct HipPlanOptions : DynamicBenchmarkOptions<int> {
  HipPlanOptions(std::vector<int> plans, std::size_t count) : DynamicBenchmarkOptions<int>(std::move(plans), count) {}
  // timings of another geometry (or pass) say nothing about this one: start again
  void bind(const flhip_conv_desc& d, int pass) {
    if (bound && pass == boundPass && std::memcmp(&d, &key, sizeof(d)) == 0) return;
    reset();
    key = d;
    boundPass = pass;
    bound = true;
  }
  flhip_conv_desc key{};
  int boundPass = -1;
  bool bound = false;
};

// Runs one backward pass under a benchmark: `run(plan)` enqueues the pass with that plan and returns the library's
// status.  With complete timings the winner runs (benchmark mode on or off); while timings are being taken (mode on)
// the current option runs inside audit(), and an option the library declines is struck out and the default rule
// runs in its place, so that the call still produces its result; otherwise the default rule.
template <typename Run>
void runPlanned(const std::shared_ptr<DynamicBenchmark>& bench, const flhip_conv_desc& d, int pass, const Run& run,
                void (*checkRc)(int)) {
  if (!bench) {
    checkRc(run(-1));
    return;
  }
  auto opts = bench->getOptions<HipPlanOptions>();
  opts->bind(d, pass);
  if (!opts->timingsComplete() && !DynamicBenchmark::getBenchmarkMode()) {
    checkRc(run(-1));
    return;
  }
  bench->audit([&] {
    // the options list is shared by the two passes; a number past this pass's own list counts as declined
    const int option = opts->currentOption();
    const int rc = option < flhip_conv2d_plan_count(pass) ? run(option) : FLHIP_DECLINED;
    if (rc == FLHIP_DECLINED) {
      opts->penalise();
      checkRc(run(-1));
    } else {
      checkRc(rc);
    }
  });
}
}  // namespace

std::shared_ptr<DynamicBenchmark> HipAutogradExtension::createBenchmarkOptions() {
  std::vector<int> plans{-1};
  const int count = std::max(flhip_conv2d_plan_count(FLHIP_CONV_BWD_DATA), flhip_conv2d_plan_count(FLHIP_CONV_BWD_FILTER));
  for (int i = 0; i < count; ++i) plans.push_back(i);
  return std::make_shared<DynamicBenchmark>(std::make_shared<HipPlanOptions>(std::move(plans), kPlanBenchCount));
}

Tensor HipAutogradExtension::workspace(size_t bytes) {
  if (bytes == 0) return Tensor();
  if (ws_.bytes() < bytes) ws_ = Tensor({(Dim)bytes}, dtype::u8);
  return ws_;
}

bool HipAutogradExtension::isDataTypeSupported(const dtype& type) const {
  return type == dtype::f32 || type == dtype::bf16 || type == dtype::f16;
}

// ---- conv2d -------------------------------------------------------------------
Tensor HipAutogradExtension::conv2d(const Tensor& input, const Tensor& weights, const Tensor& bias,
                                    const int sx, const int sy, const int px, const int py,
                                    const int dx, const int dy, const int groups,
                                    std::shared_ptr<detail::AutogradPayload> autogradPayload) {
  if (input.type() != weights.type())
    throw std::invalid_argument("conv2d: input and weights must have the same type");
  detail::OpScope scope("conv2d");
  const int tag = dtypeTag(input.type(), "conv2d");
  flhip_conv_desc d = convDesc(input.shape(), weights, sx, sy, px, py, dx, dy, groups, tag, "conv2d");
  int32_t OH = 0, OW = 0;
  check(flhip_conv2d_out_dims(&d, &OH, &OW));
  const bool hasBias = bias.elements() > 0;       // onednn/Conv2D.cpp:71,189
  if (hasBias && bias.elements() != d.K)
    throw std::invalid_argument("conv2d: bias must have one element per output channel");
  const Tensor b = asF32(bias);
  Tensor output({OW, OH, d.K, d.N}, input.type());
  const size_t wsBytes = flhip_conv2d_workspace_bytes(&d, FLHIP_CONV_FWD);
  // a tape is being recorded and this layer's forward pass gathers its input: the pass gets a workspace of its
  // own, which the payload keeps for the filter gradient (the shared one is overwritten by the next layer)
  const bool keep = autogradPayload != nullptr && wsBytes > 0 && flhip_conv2d_gathered_bytes(&d) > 0;
  Tensor ws = keep ? Tensor({(Dim)wsBytes}, dtype::u8) : workspace(wsBytes);
  if (keep) {
    auto payload = std::make_shared<HipConv2DPayload>();
    payload->gathered = ws;
    autogradPayload->data = payload;
  }
  DevicePtr xp(input), wp(weights), bp(b), yp(output), wsp(ws);
  check(flhip_conv2d_fwd(&d, xp.get(), wp.get(), static_cast<const float*>(bp.get()), yp.get(),
                         wsp.get(), wsBytes, hipBackendStream()));
  // event: inputs {input, weights, bias}, outputs {output}, ints {sx, sy, px, py, dx, dy, groups}
  if (scope.on()) scope.done({input, weights, b}, {output}, {sx, sy, px, py, dx, dy, groups});
  return output;
}

Tensor HipAutogradExtension::conv2dBackwardData(const Tensor& gradOutput, const Tensor& input,
                                                const Tensor& weight, const int sx, const int sy,
                                                const int px, const int py, const int dx,
                                                const int dy, const int groups,
                                                std::shared_ptr<DynamicBenchmark> dataGradBenchmark,
                                                std::shared_ptr<detail::AutogradPayload>) {
  if (gradOutput.type() != weight.type())
    throw std::invalid_argument("conv2dBackwardData: gradOutput and weights must have the same type");
  detail::OpScope scope("conv2dBackwardData");
  const int tag = dtypeTag(gradOutput.type(), "conv2dBackwardData");
  flhip_conv_desc d =
      convDesc(input.shape(), weight, sx, sy, px, py, dx, dy, groups, tag, "conv2dBackwardData");
  int32_t OH = 0, OW = 0;
  check(flhip_conv2d_out_dims(&d, &OH, &OW));
  if (gradOutput.shape() != Shape({OW, OH, d.K, d.N}))
    throw std::invalid_argument("conv2dBackwardData: gradOutput shape does not match the geometry");
  Tensor gradInput(input.shape(), gradOutput.type());   // onednn/Conv2D.cpp:285
  const size_t wsBytes = flhip_conv2d_workspace_bytes(&d, FLHIP_CONV_BWD_DATA);
  Tensor ws = workspace(wsBytes);
  DevicePtr gp(gradOutput), wp(weight), op(gradInput), wsp(ws);
  runPlanned(dataGradBenchmark, d, FLHIP_CONV_BWD_DATA, [&](int plan) {
    return flhip_conv2d_bwd_data_plan(&d, gp.get(), wp.get(), op.get(), wsp.get(), wsBytes, plan, hipBackendStream());
  }, &check);
  // event: inputs {gradOutput, weights}, outputs {gradInput}, ints as conv2d
  if (scope.on()) scope.done({gradOutput, weight}, {gradInput}, {sx, sy, px, py, dx, dy, groups});
  return gradInput;
}

Tensor HipAutogradExtension::conv2dBackwardDataAdd(const Tensor& gradOutput, const Tensor& input,
                                                   const Tensor& weight, const Tensor& addend, const int sx,
                                                   const int sy, const int px, const int py, const int dx,
                                                   const int dy, const int groups) {
  if (gradOutput.type() != weight.type() || addend.type() != gradOutput.type())
    throw std::invalid_argument("conv2dBackwardDataAdd: gradOutput, weights and addend must have the same type");
  if (addend.shape() != input.shape())
    throw std::invalid_argument("conv2dBackwardDataAdd: addend must have the input's shape");
  detail::OpScope scope("conv2dBackwardDataAdd");
  const int tag = dtypeTag(gradOutput.type(), "conv2dBackwardDataAdd");
  flhip_conv_desc d =
      convDesc(input.shape(), weight, sx, sy, px, py, dx, dy, groups, tag, "conv2dBackwardDataAdd");
  int32_t OH = 0, OW = 0;
  check(flhip_conv2d_out_dims(&d, &OH, &OW));
  if (gradOutput.shape() != Shape({OW, OH, d.K, d.N}))
    throw std::invalid_argument("conv2dBackwardDataAdd: gradOutput shape does not match the geometry");
  Tensor gradInput(input.shape(), gradOutput.type());
  const size_t wsBytes = flhip_conv2d_workspace_bytes(&d, FLHIP_CONV_BWD_DATA);
  Tensor ws = workspace(wsBytes);
  DevicePtr gp(gradOutput), wp(weight), ap(addend), op(gradInput), wsp(ws);
  check(flhip_conv2d_bwd_data_add(&d, gp.get(), wp.get(), ap.get(), op.get(), wsp.get(), wsBytes,
                                  hipBackendStream()));
  // event: inputs {gradOutput, weights, addend}, outputs {gradInput}, ints as conv2d
  if (scope.on()) scope.done({gradOutput, weight, addend}, {gradInput}, {sx, sy, px, py, dx, dy, groups});
  return gradInput;
}

std::pair<Tensor, Tensor> HipAutogradExtension::conv2dBackwardFilterBias(
    const Tensor& gradOutput, const Tensor& input, const Tensor& weights, const Tensor& bias,
    const int sx, const int sy, const int px, const int py, const int dx, const int dy,
    const int groups, std::shared_ptr<DynamicBenchmark> filterBench, std::shared_ptr<DynamicBenchmark>,
    std::shared_ptr<detail::AutogradPayload> autogradPayload) {
  if (gradOutput.type() != input.type())
    throw std::invalid_argument("conv2dBackwardFilterBias: gradOutput and input must have the same type");
  detail::OpScope scope("conv2dBackwardFilterBias");
  const int tag = dtypeTag(input.type(), "conv2dBackwardFilterBias");
  flhip_conv_desc d = convDesc(input.shape(), weights, sx, sy, px, py, dx, dy, groups, tag,
                               "conv2dBackwardFilterBias");
  int32_t OH = 0, OW = 0;
  check(flhip_conv2d_out_dims(&d, &OH, &OW));
  if (gradOutput.shape() != Shape({OW, OH, d.K, d.N}))
    throw std::invalid_argument("conv2dBackwardFilterBias: gradOutput shape does not match the geometry");
  // gradients are produced in fp32 (for bf16 storage: the master-weight precision)
  Tensor gradWeights(weights.shape(), dtype::f32);
  // the bias gradient comes from the same pass iff a bias was passed
  // (onednn/Conv2D.cpp:411-415); the caller passes an empty one when it is not
  // needed (flashlight/fl/autograd/Functions.cpp:1391-1395)
  Tensor gradBias;
  if (!bias.isEmpty()) gradBias = Tensor(bias.shape(), dtype::f32);
  const size_t wsBytes = flhip_conv2d_workspace_bytes(&d, FLHIP_CONV_BWD_FILTER);
  Tensor ws = workspace(wsBytes);
  DevicePtr xp(input), gp(gradOutput), dwp(gradWeights), dbp(gradBias), wsp(ws);
  std::shared_ptr<HipConv2DPayload> kept;
  if (autogradPayload && autogradPayload->data) kept = std::dynamic_pointer_cast<HipConv2DPayload>(autogradPayload->data);
  const size_t gatheredBytes = kept ? flhip_conv2d_gathered_bytes(&d) : 0;
  // the forward pass's gathered input in place of x where the library still takes it for this geometry (a
  // process-wide option changed between the two passes can withdraw it: then, as without a payload, from x)
  int rc = FLHIP_INVALID_ARGUMENT;
  if (kept && gatheredBytes > 0 && kept->gathered.bytes() >= gatheredBytes) {
    DevicePtr kp(kept->gathered);
    rc = flhip_conv2d_bwd_filter_gathered(&d, kp.get(), gp.get(), static_cast<float*>(dwp.get()),
                                          static_cast<float*>(dbp.get()), wsp.get(), wsBytes,
                                          hipBackendStream());
    if (rc != FLHIP_OK && rc != FLHIP_INVALID_ARGUMENT) check(rc);
  }
  // (the bias gradient comes out of the same pass: the bias benchmark of the reference's closure has nothing to choose)
  if (rc != FLHIP_OK)
    runPlanned(filterBench, d, FLHIP_CONV_BWD_FILTER, [&](int plan) {
      return flhip_conv2d_bwd_filter_plan(&d, xp.get(), gp.get(), static_cast<float*>(dwp.get()),
                                          static_cast<float*>(dbp.get()), wsp.get(), wsBytes, plan, hipBackendStream());
    }, &check);
  // event: inputs {gradOutput, input}, outputs {gradWeights, gradBias (may be empty)}, ints as conv2d
  if (scope.on()) scope.done({gradOutput, input}, {gradWeights, gradBias}, {sx, sy, px, py, dx, dy, groups});
  return {gradWeights, gradBias};
}

// ---- pool2d -------------------------------------------------------------------
namespace {
flhip_pool_desc poolDesc(const Shape& in, int wx, int wy, int sx, int sy, int px, int py,
                         PoolingMode mode, int tag) {
  // missing trailing dimensions count as 1 (onednn/Pool2D.cpp:95-98)
  flhip_pool_desc d{};
  d.W = (int)in.dim(0);
  d.H = in.ndim() > 1 ? (int)in.dim(1) : 1;
  d.C = in.ndim() > 2 ? (int)in.dim(2) : 1;
  d.N = in.ndim() > 3 ? (int)in.dim(3) : 1;
  d.wx = wx; d.wy = wy; d.sx = sx; d.sy = sy; d.px = px; d.py = py;
  d.mode = (int)mode;
  d.dtype = tag;
  return d;
}
}  // namespace

Tensor HipAutogradExtension::pool2d(const Tensor& input, const int wx, const int wy, const int sx,
                                    const int sy, const int px, const int py,
                                    const PoolingMode mode,
                                    std::shared_ptr<detail::AutogradPayload> autogradPayload) {
  if (input.ndim() < 1 || input.ndim() > 4)
    throw std::invalid_argument("pool2d: input must have 1 to 4 dimensions");
  detail::OpScope scope("pool2d");
  const bool train = autogradPayload != nullptr;    // onednn/Pool2D.cpp:88
  flhip_pool_desc d = poolDesc(input.shape(), wx, wy, sx, sy, px, py, mode, dtypeTag(input.type(), "pool2d"));
  int32_t OH = 0, OW = 0;
  check(flhip_pool2d_out_dims(&d, &OH, &OW));
  Tensor output({OW, OH, d.C, d.N}, input.type());
  auto payload = std::make_shared<HipPool2DPayload>();
  if (train && mode == PoolingMode::MAX) payload->argmax = Tensor({OW, OH, d.C, d.N}, dtype::u8);
  if (train) autogradPayload->data = payload;
  DevicePtr xp(input), yp(output), ap(payload->argmax);
  check(flhip_pool2d_fwd(&d, xp.get(), yp.get(), static_cast<uint8_t*>(ap.get()), hipBackendStream()));
  // event: inputs {input}, outputs {output, argmax (may be empty)}, ints {wx, wy, sx, sy, px, py, mode}
  if (scope.on()) scope.done({input}, {output, payload->argmax}, {wx, wy, sx, sy, px, py, (int)mode});
  return output;
}

Tensor HipAutogradExtension::pool2dBackward(const Tensor& gradOutput, const Tensor& input,
                                            const Tensor&, const int wx, const int wy,
                                            const int sx, const int sy, const int px, const int py,
                                            const PoolingMode mode,
                                            std::shared_ptr<detail::AutogradPayload> autogradPayload) {
  detail::OpScope scope("pool2dBackward");
  if (!autogradPayload || !autogradPayload->data)   // onednn/Pool2D.cpp:190-193
    throw std::invalid_argument("HipAutogradExtension::pool2dBackward given null or empty payload");
  auto payload = std::dynamic_pointer_cast<HipPool2DPayload>(autogradPayload->data);
  if (!payload) throw std::invalid_argument("pool2dBackward: payload of another operation");
  flhip_pool_desc d =
      poolDesc(input.shape(), wx, wy, sx, sy, px, py, mode, dtypeTag(gradOutput.type(), "pool2dBackward"));
  int32_t OH = 0, OW = 0;
  check(flhip_pool2d_out_dims(&d, &OH, &OW));
  if (gradOutput.elements() != (Dim)OW * OH * d.C * d.N)
    throw std::invalid_argument("pool2dBackward: gradOutput shape does not match the geometry");
  // the reference allocates f32 whatever the input type (onednn/Pool2D.cpp:197),
  // which its own caller cannot add to a non-f32 gradient; here the gradient has
  // the type of gradOutput
  Tensor gradInput(input.shape(), gradOutput.type());
  DevicePtr gp(gradOutput), ap(payload->argmax), op(gradInput);
  check(flhip_pool2d_bwd(&d, gp.get(), static_cast<const uint8_t*>(ap.get()), op.get(),
                         hipBackendStream()));
  // event: inputs {gradOutput, argmax}, outputs {gradInput}, ints as pool2d
  if (scope.on()) scope.done({gradOutput, payload->argmax}, {gradInput}, {wx, wy, sx, sy, px, py, (int)mode});
  return gradInput;
}

// ---- batchnorm ------------------------------------------------------------------
Tensor HipAutogradExtension::batchnorm(Tensor& saveMean, Tensor& saveVar, const Tensor& input,
                                       const Tensor& weight, const Tensor& bias,
                                       Tensor& runningMean, Tensor& runningVar,
                                       const std::vector<int>& axes, const bool train,
                                       const double momentum, const double epsilon,
                                       std::shared_ptr<detail::AutogradPayload> autogradPayload) {
  detail::OpScope scope("batchnorm");
  const int tag = dtypeTag(input.type(), "batchnorm");
  flhip_bn_desc d = bnDesc(input, axes, tag);
  const Dim nfeat = (Dim)d.C;
  for (const Tensor* t : {&weight, &bias, static_cast<const Tensor*>(&runningMean),
                          static_cast<const Tensor*>(&runningVar)})
    if (!t->isEmpty() && t->elements() != nfeat)
      throw std::invalid_argument("batchnorm: parameters must have one element per feature");
  // empty running statistics are created (onednn/BatchNorm.cpp:116-122); they stay fp32
  if (runningVar.isEmpty()) runningVar = Tensor::full({nfeat}, 1., dtype::f32);
  if (runningMean.isEmpty()) runningMean = Tensor::full({nfeat}, 0., dtype::f32);
  if (runningMean.type() != dtype::f32 || runningVar.type() != dtype::f32)
    throw std::invalid_argument("batchnorm: running statistics must be f32");
  const Tensor gamma = asF32(weight), beta = asF32(bias);   // empty = no affine (:136-139)
  Tensor output(input.shape(), input.type());
  DevicePtr xp(input), gp(gamma), bp(beta), yp(output), rmp(runningMean), rvp(runningVar);
  if (!train) {
    check(flhip_bn_fwd_infer(&d, xp.get(), static_cast<const float*>(gp.get()),
                             static_cast<const float*>(bp.get()),
                             static_cast<const float*>(rmp.get()),
                             static_cast<const float*>(rvp.get()), epsilon, yp.get(),
                             hipBackendStream()));
    if (scope.on())
      scope.done({input, gamma, beta, runningMean, runningVar}, {output}, {d.outer, d.C, d.inner, 0}, {momentum, epsilon});
    return output;
  }
  // like the cuDNN extension (cudnn/BatchNorm.cpp:138-162): saveMean holds the batch
  // mean, saveVar the inverse standard deviation, both f32
  saveMean = Tensor({nfeat}, dtype::f32);
  saveVar = Tensor({nfeat}, dtype::f32);
  const size_t wsBytes = flhip_bn_workspace_bytes(&d);
  Tensor ws = workspace(wsBytes);
  DevicePtr smp(saveMean), sip(saveVar), wsp(ws);
  check(flhip_bn_fwd_train(&d, xp.get(), static_cast<const float*>(gp.get()),
                           static_cast<const float*>(bp.get()), yp.get(),
                           static_cast<float*>(smp.get()), static_cast<float*>(sip.get()),
                           static_cast<float*>(rmp.get()), static_cast<float*>(rvp.get()), momentum,
                           epsilon, wsp.get(), wsBytes, hipBackendStream()));
  if (autogradPayload) {
    auto payload = std::make_shared<HipBatchNormPayload>();
    payload->saveMean = saveMean;
    payload->saveInvStd = saveVar;
    autogradPayload->data = payload;
  }
  // event: inputs {input, gamma, beta, runningMean, runningVar (both after the update)}, outputs {output, saveMean,
  // saveInvStd}, ints {outer, features, inner, train}, reals {momentum, epsilon}
  if (scope.on())
    scope.done({input, gamma, beta, runningMean, runningVar}, {output, saveMean, saveVar}, {d.outer, d.C, d.inner, 1},
               {momentum, epsilon});
  return output;
}

std::tuple<Tensor, Tensor, Tensor> HipAutogradExtension::batchnormBackward(
    const Tensor& gradOutput, const Tensor& saveMean, const Tensor& saveVar, const Tensor& input,
    const Tensor& weight, const std::vector<int>& axes, const bool train, const float,
    std::shared_ptr<detail::AutogradPayload> autogradPayload) {
  detail::OpScope scope("batchnormBackward");
  if (!train)   // cudnn/BatchNorm.cpp:196-199
    throw std::logic_error("HipAutogradExtension::batchnormBackward: only train mode has a backward pass");
  Tensor mean = saveMean, invstd = saveVar;
  if (autogradPayload && autogradPayload->data) {
    auto payload = std::dynamic_pointer_cast<HipBatchNormPayload>(autogradPayload->data);
    if (!payload) throw std::invalid_argument("batchnormBackward: payload of another operation");
    mean = payload->saveMean;
    invstd = payload->saveInvStd;
  }
  if (mean.isEmpty() || invstd.isEmpty())   // onednn/BatchNorm.cpp:212-215
    throw std::invalid_argument("HipAutogradExtension::batchnormBackward given null or empty payload");
  if (gradOutput.type() != input.type() || gradOutput.shape() != input.shape())
    throw std::invalid_argument("batchnormBackward: gradOutput must match the input");
  flhip_bn_desc d = bnDesc(input, axes, dtypeTag(input.type(), "batchnormBackward"));
  const Dim nfeat = (Dim)d.C;
  const Tensor gamma = asF32(weight);
  Tensor gradInput(input.shape(), input.type());
  Tensor gradWeight({nfeat}, dtype::f32), gradBias({nfeat}, dtype::f32);
  const size_t wsBytes = flhip_bn_workspace_bytes(&d);
  Tensor ws = workspace(wsBytes);
  DevicePtr xp(input), dyp(gradOutput), gp(gamma), mp(mean), ip(invstd), dxp(gradInput),
      dgp(gradWeight), dbp(gradBias), wsp(ws);
  check(flhip_bn_bwd(&d, xp.get(), dyp.get(), static_cast<const float*>(gp.get()),
                     static_cast<const float*>(mp.get()), static_cast<const float*>(ip.get()),
                     dxp.get(), static_cast<float*>(dgp.get()), static_cast<float*>(dbp.get()),
                     wsp.get(), wsBytes, hipBackendStream()));
  // event: inputs {gradOutput, input, gamma, saveMean, saveInvStd}, outputs {gradInput, gradWeight, gradBias},
  // ints {outer, features, inner}
  if (scope.on())
    scope.done({gradOutput, input, gamma, mean, invstd}, {gradInput, gradWeight, gradBias}, {d.outer, d.C, d.inner});
  return std::make_tuple(gradInput, gradWeight, gradBias);   // always all three (:278)
}

// ---- batch norm fused with the residual add and the ReLU ----------------------------------------
Tensor HipAutogradExtension::batchnormRelu(Tensor& saveMean, Tensor& saveVar, const Tensor& input,
                                           const Tensor& weight, const Tensor& bias, Tensor& runningMean,
                                           Tensor& runningVar, const std::vector<int>& axes,
                                           const double momentum, const double epsilon, const Tensor& residual,
                                           std::shared_ptr<detail::AutogradPayload> autogradPayload) {
  detail::OpScope scope("batchnormRelu");
  const int tag = dtypeTag(input.type(), "batchnormRelu");
  flhip_bn_desc d = bnDesc(input, axes, tag);
  const Dim nfeat = (Dim)d.C;
  for (const Tensor* t : {&weight, &bias, static_cast<const Tensor*>(&runningMean),
                          static_cast<const Tensor*>(&runningVar)})
    if (!t->isEmpty() && t->elements() != nfeat)
      throw std::invalid_argument("batchnormRelu: parameters must have one element per feature");
  if (!residual.isEmpty() && (residual.type() != input.type() || residual.shape() != input.shape()))
    throw std::invalid_argument("batchnormRelu: the residual must match the input");
  if (runningVar.isEmpty()) runningVar = Tensor::full({nfeat}, 1., dtype::f32);
  if (runningMean.isEmpty()) runningMean = Tensor::full({nfeat}, 0., dtype::f32);
  if (runningMean.type() != dtype::f32 || runningVar.type() != dtype::f32)
    throw std::invalid_argument("batchnormRelu: running statistics must be f32");
  const Tensor gamma = asF32(weight), beta = asF32(bias);
  Tensor output(input.shape(), input.type());
  saveMean = Tensor({nfeat}, dtype::f32);
  saveVar = Tensor({nfeat}, dtype::f32);
  const size_t wsBytes = flhip_bn_workspace_bytes(&d);
  Tensor ws = workspace(wsBytes);
  // with a tape to feed, the ReLU's mask goes along as bits: the backward pass then reads a quarter
  // of a byte per element instead of the whole result
  const size_t maskBytes = autogradPayload ? flhip_bn_act_mask_bytes(&d) : 0;
  Tensor mask = maskBytes ? Tensor({(Dim)maskBytes}, dtype::u8) : Tensor();
  DevicePtr xp(input), gp(gamma), bp(beta), rp(residual), yp(output), rmp(runningMean), rvp(runningVar),
      smp(saveMean), sip(saveVar), wsp(ws), mkp(mask);
  if (maskBytes)
    check(flhip_bn_act_fwd_train_mask(&d, xp.get(), static_cast<const float*>(gp.get()),
                                      static_cast<const float*>(bp.get()), rp.get(), 1, yp.get(), mkp.get(),
                                      static_cast<float*>(smp.get()), static_cast<float*>(sip.get()),
                                      static_cast<float*>(rmp.get()), static_cast<float*>(rvp.get()), momentum,
                                      epsilon, wsp.get(), wsBytes, hipBackendStream()));
  else
    check(flhip_bn_act_fwd_train(&d, xp.get(), static_cast<const float*>(gp.get()),
                                 static_cast<const float*>(bp.get()), rp.get(), 1, yp.get(),
                                 static_cast<float*>(smp.get()), static_cast<float*>(sip.get()),
                                 static_cast<float*>(rmp.get()), static_cast<float*>(rvp.get()), momentum, epsilon,
                                 wsp.get(), wsBytes, hipBackendStream()));
  if (autogradPayload) {
    auto payload = std::make_shared<HipBatchNormPayload>();
    payload->saveMean = saveMean;
    payload->saveInvStd = saveVar;
    payload->reluMask = mask;
    autogradPayload->data = payload;
  }
  // event: inputs {input, gamma, beta, runningMean, runningVar, residual (may be empty)}, outputs {output, saveMean,
  // saveInvStd}, ints {outer, features, inner, train = 1}, reals {momentum, epsilon}
  if (scope.on())
    scope.done({input, gamma, beta, runningMean, runningVar, residual}, {output, saveMean, saveVar},
               {d.outer, d.C, d.inner, 1}, {momentum, epsilon});
  return output;
}

std::tuple<Tensor, Tensor, Tensor, Tensor> HipAutogradExtension::batchnormReluBackward(
    const Tensor& gradOutput, const Tensor& output, const Tensor& saveMean, const Tensor& saveVar,
    const Tensor& input, const Tensor& weight, const std::vector<int>& axes, const bool wantResidualGrad,
    std::shared_ptr<detail::AutogradPayload> autogradPayload) {
  detail::OpScope scope("batchnormReluBackward");
  Tensor mean = saveMean, invstd = saveVar, mask;
  if (autogradPayload && autogradPayload->data) {
    auto payload = std::dynamic_pointer_cast<HipBatchNormPayload>(autogradPayload->data);
    if (!payload) throw std::invalid_argument("batchnormReluBackward: payload of another operation");
    mean = payload->saveMean;
    invstd = payload->saveInvStd;
    mask = payload->reluMask;
  }
  if (mean.isEmpty() || invstd.isEmpty())
    throw std::invalid_argument("HipAutogradExtension::batchnormReluBackward given null or empty payload");
  if (gradOutput.type() != input.type() || gradOutput.shape() != input.shape() ||
      output.type() != input.type() || output.shape() != input.shape())
    throw std::invalid_argument("batchnormReluBackward: gradOutput and output must match the input");
  flhip_bn_desc d = bnDesc(input, axes, dtypeTag(input.type(), "batchnormReluBackward"));
  const Dim nfeat = (Dim)d.C;
  const Tensor gamma = asF32(weight);
  Tensor gradInput(input.shape(), input.type());
  Tensor gradResidual = wantResidualGrad ? Tensor(input.shape(), input.type()) : Tensor();
  Tensor gradWeight({nfeat}, dtype::f32), gradBias({nfeat}, dtype::f32);
  const size_t wsBytes = flhip_bn_workspace_bytes(&d);
  Tensor ws = workspace(wsBytes);
  DevicePtr xp(input), dyp(gradOutput), yp(output), gp(gamma), mp(mean), ip(invstd), dxp(gradInput),
      drp(gradResidual), dgp(gradWeight), dbp(gradBias), wsp(ws), mkp(mask);
  if (!mask.isEmpty()) {
    if ((size_t)mask.elements() != flhip_bn_act_mask_bytes(&d))
      throw std::invalid_argument("batchnormReluBackward: payload of another call");
    check(flhip_bn_act_bwd_mask(&d, xp.get(), dyp.get(), mkp.get(), static_cast<const float*>(gp.get()),
                                static_cast<const float*>(mp.get()), static_cast<const float*>(ip.get()), dxp.get(),
                                drp.get(), static_cast<float*>(dgp.get()), static_cast<float*>(dbp.get()), wsp.get(),
                                wsBytes, hipBackendStream()));
  } else {
    check(flhip_bn_act_bwd(&d, xp.get(), dyp.get(), yp.get(), static_cast<const float*>(gp.get()),
                           static_cast<const float*>(mp.get()), static_cast<const float*>(ip.get()), dxp.get(),
                           drp.get(), static_cast<float*>(dgp.get()), static_cast<float*>(dbp.get()), wsp.get(),
                           wsBytes, hipBackendStream()));
  }
  // event: inputs {gradOutput, input, gamma, saveMean, saveInvStd, output}, outputs {gradInput, gradWeight,
  // gradBias, gradResidual (may be empty)}, ints {outer, features, inner}
  if (scope.on())
    scope.done({gradOutput, input, gamma, mean, invstd, output}, {gradInput, gradWeight, gradBias, gradResidual},
               {d.outer, d.C, d.inner});
  return std::make_tuple(gradInput, gradWeight, gradBias, gradResidual);
}

// ---- rnn (flashlight/fl/autograd/tensor/backend/cudnn/RNN.cpp:62-375) -------------------
namespace {
struct HipRnnPayload : detail::AutogradPayloadData {
  Tensor reserve;   // states and gate activations of the forward pass
  unsigned long long seed = 0;   // of the dropout mask between layers
};

flhip_rnn_desc rnnDesc(const Tensor& input, int hiddenSize, int numLayers, RnnMode mode, bool bidirectional,
                       float dropProb, unsigned long long seed) {
  if (input.type() != dtype::f32) throw std::runtime_error("HipAutogradExtension::rnn: f32 only");
  flhip_rnn_desc d{};
  d.input_size = (int32_t)input.dim(0);
  d.batch = input.ndim() < 2 ? 1 : (int32_t)input.dim(1);
  d.seq_len = input.ndim() < 3 ? 1 : (int32_t)input.dim(2);
  d.hidden_size = hiddenSize;
  d.num_layers = numLayers;
  d.bidirectional = bidirectional ? 1 : 0;
  d.mode = (int32_t)mode;
  d.dtype = FLHIP_F32;
  if (!(dropProb >= 0.f && dropProb < 1.f)) throw std::invalid_argument("rnn: dropout must be in [0, 1)");
  d.dropout = numLayers > 1 ? dropProb : 0.f;   // between layers only (RNN.cpp:83-90)
  d.seed_lo = (uint32_t)seed;
  d.seed_hi = (uint32_t)(seed >> 32);
  return d;
}
}  // namespace

unsigned long long nextSeed();   // Modules.cpp: the process-wide generator

std::tuple<Tensor, Tensor, Tensor> HipAutogradExtension::rnn(
    const Tensor& input, const Tensor& hiddenState, const Tensor& cellState, const Tensor& weights,
    const int hiddenSize, const int numLayers, const RnnMode mode, const bool bidirectional,
    const float dropProb, std::shared_ptr<detail::AutogradPayload> autogradPayload) {
  detail::OpScope scope("rnn");
  if (input.isEmpty()) throw std::runtime_error("HipAutogradExtension::rnn: empty input");
  for (const Tensor* t : {&hiddenState, &cellState, &weights})
    if (!t->isEmpty() && t->type() != input.type())
      throw std::invalid_argument("rnn doesn't support binary operations with Tensors of different types");
  if (input.type() == dtype::bf16 || input.type() == dtype::f16) {
    const dtype lo = input.type();
    // 16-bit storage (the reference: half tensors, RNN.cpp:45): the device kernels are fp32, so the
    // tensors are widened at the boundary and the results rounded once on the way out
    auto up = [](const Tensor& t) { return t.isEmpty() ? t : t.astype(dtype::f32); };
    Tensor y, hy, cy;
    std::tie(y, hy, cy) = rnn(up(input), up(hiddenState), up(cellState), up(weights), hiddenSize, numLayers, mode,
                              bidirectional, dropProb, autogradPayload);
    return std::make_tuple(y.astype(lo), hy.astype(lo), cy.isEmpty() ? cy : cy.astype(lo));
  }
  const unsigned long long seed = dropProb > 0.f ? nextSeed() : 0ull;
  const flhip_rnn_desc d = rnnDesc(input, hiddenSize, numLayers, mode, bidirectional, dropProb, seed);
  const Dim totalLayers = numLayers * (bidirectional ? 2 : 1), outSize = hiddenSize * (bidirectional ? 2 : 1);
  // RNN.cpp:97-113
  if (!hiddenState.isEmpty()) {
    const Dim hb = hiddenState.ndim() < 2 ? 1 : hiddenState.dim(1), hl = hiddenState.ndim() < 3 ? 1 : hiddenState.dim(2);
    if (!(hiddenState.dim(0) == hiddenSize && hb == d.batch && hl == totalLayers))
      throw std::invalid_argument("invalid hidden state dims for RNN");
  }
  if (!cellState.isEmpty() &&
      !(mode == RnnMode::LSTM && cellState.ndim() == 3 && cellState.dim(0) == hiddenSize &&
        cellState.dim(1) == d.batch && cellState.dim(2) == totalLayers))
    throw std::invalid_argument("invalid cell state dims for RNN");
  if ((size_t)weights.elements() != flhip_rnn_param_count(&d) || flhip_rnn_param_count(&d) == 0)
    throw std::invalid_argument("invalid # of parameters or wrong input shape for RNN");   // :123-133

  Tensor y({outSize, d.batch, d.seq_len}, input.type());
  Tensor hy({(Dim)hiddenSize, d.batch, totalLayers}, input.type());
  Tensor cy = mode == RnnMode::LSTM ? Tensor(hy.shape(), input.type()) : Tensor();
  const size_t resBytes = flhip_rnn_reserve_bytes(&d), wsBytes = flhip_rnn_workspace_bytes(&d);
  Tensor reserve({(Dim)resBytes}, dtype::u8);
  Tensor ws = workspace(wsBytes);
  DevicePtr xp(input), hp(hiddenState), cp(cellState), wp(weights), yp(y), hyp(hy), cyp(cy), rp(reserve), wsp(ws);
  check(flhip_rnn_fwd(&d, xp.get(), hp.get(), cp.get(), wp.get(), yp.get(), hyp.get(), cyp.get(), rp.get(),
                      resBytes, wsp.get(), wsBytes, hipBackendStream()));
  if (autogradPayload) {
    auto payload = std::make_shared<HipRnnPayload>();
    payload->reserve = reserve;
    payload->seed = seed;
    autogradPayload->data = payload;
  }
  if (scope.on()) scope.done({input, hiddenState, cellState, weights}, {y, hy, cy}, {hiddenSize, numLayers, (int)mode, bidirectional});
  return std::make_tuple(y, hy, cy);
}

std::tuple<Tensor, Tensor, Tensor, Tensor> HipAutogradExtension::rnnBackward(
    const Tensor& input, const Tensor& hiddenState, const Tensor& cellState, const Tensor& weights,
    const std::shared_ptr<detail::RNNGradData> gradData, const Tensor& output, const int numLayers,
    const int hiddenSize, const RnnMode mode, const bool bidirectional, const float dropProb,
    std::shared_ptr<detail::AutogradPayload> autogradPayload) {
  detail::OpScope scope("rnnBackward");
  if (!autogradPayload || !autogradPayload->data)   // RNN.cpp:246-249
    throw std::invalid_argument("HipAutogradExtension::rnnBackward given null or empty autograd payload");
  auto payload = std::dynamic_pointer_cast<HipRnnPayload>(autogradPayload->data);
  if (!payload) throw std::invalid_argument("rnnBackward: payload of another operation");
  if (!gradData) throw std::invalid_argument("rnnBackward: no gradient data");
  if (input.type() == dtype::bf16 || input.type() == dtype::f16) {
    const dtype lo = input.type();
    auto up = [](const Tensor& t) { return t.isEmpty() ? t : t.astype(dtype::f32); };
    auto wide = std::make_shared<detail::RNNGradData>();
    wide->dy = up(gradData->dy);
    wide->dhy = up(gradData->dhy);
    wide->dcy = up(gradData->dcy);
    Tensor dx, dhx, dcx, dw;
    std::tie(dx, dhx, dcx, dw) = rnnBackward(up(input), up(hiddenState), up(cellState), up(weights), wide, up(output),
                                            numLayers, hiddenSize, mode, bidirectional, dropProb, autogradPayload);
    return std::make_tuple(dx.astype(lo), dhx.astype(lo), dcx.isEmpty() ? dcx : dcx.astype(lo), dw.astype(lo));
  }
  const flhip_rnn_desc d = rnnDesc(input, hiddenSize, numLayers, mode, bidirectional, dropProb, payload->seed);
  const Dim totalLayers = numLayers * (bidirectional ? 2 : 1);
  // output gradients nobody produced are zero (RNN.cpp:262-275)
  for (const Tensor* t : {&gradData->dy, &gradData->dhy, &gradData->dcy})
    if (!t->isEmpty() && t->type() != dtype::f32) throw std::runtime_error("rnnBackward: f32 only");
  if (!gradData->dy.isEmpty() && gradData->dy.elements() != output.elements())
    throw std::invalid_argument("rnnBackward: gradient of the output has the wrong size");
  Tensor dx(input.shape(), input.type());
  Tensor dhx({(Dim)hiddenSize, d.batch, totalLayers}, input.type());
  Tensor dcx = mode == RnnMode::LSTM ? Tensor(dhx.shape(), input.type()) : Tensor();
  Tensor dw(weights.shape(), weights.type());
  const size_t resBytes = flhip_rnn_reserve_bytes(&d), wsBytes = flhip_rnn_workspace_bytes(&d);
  Tensor ws = workspace(wsBytes);
  DevicePtr xp(input), wp(weights), dyp(gradData->dy), dhyp(gradData->dhy), dcyp(gradData->dcy),
      rp(payload->reserve), dxp(dx), dhxp(dhx), dcxp(dcx), dwp(dw), wsp(ws);
  check(flhip_rnn_bwd(&d, xp.get(), wp.get(), dyp.get(), dhyp.get(), mode == RnnMode::LSTM ? dcyp.get() : nullptr,
                      rp.get(), resBytes, dxp.get(), dhxp.get(), dcxp.get(), dwp.get(), wsp.get(), wsBytes,
                      hipBackendStream()));
  (void)hiddenState;
  (void)cellState;
  if (scope.on()) scope.done({input, weights, gradData->dy, gradData->dhy, gradData->dcy}, {dx, dhx, dcx, dw}, {hiddenSize, numLayers, (int)mode, bidirectional});
  return std::make_tuple(dx, dhx, dcx, dw);
}

}  // namespace fl
