/*
 * flhip.h — C ABI of the MI355X (gfx950) kernels behind Flashlight's
 * AutogradExtension operator interface.
 *
 * The reference has no C ABI for this path: its extension point is the C++
 * abstract class fl::AutogradExtension
 * (flashlight/fl/autograd/tensor/AutogradExtension.h:46-180).  Each entry point
 * below is what one virtual of that class lowers to once tensors have been
 * reduced to raw device pointers, and names the virtual it serves.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer into memory owned by the caller.
 *   - Layout: Flashlight column-major [W,H,C,N] == row-major N,C,H,W; weights
 *     [kx,ky,Cin/groups,Cout] == row-major Cout,Cin/groups,KH,KW
 *     (flashlight/fl/autograd/tensor/backend/onednn/Conv2D.cpp:69-93,171-178).
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Work
 *     is enqueued; no entry point synchronises the device.
 *   - Return value: FLHIP_OK, FLHIP_INVALID_ARGUMENT (host maps it to
 *     std::invalid_argument) or FLHIP_RUNTIME_ERROR (std::runtime_error), the two
 *     exception kinds of the reference boundary
 *     (flashlight/fl/autograd/tensor/backend/cudnn/CudnnUtils.cpp:88-99).
 *     flhip_last_error() returns the message of the calling thread's last failure.
 *   - The library allocates nothing: scratch comes in through `ws`/`ws_bytes`
 *     (size from the matching *_workspace_bytes query).
 */
#ifndef FLHIP_H
#define FLHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  FLHIP_OK = 0,
  FLHIP_INVALID_ARGUMENT = 1,
  FLHIP_RUNTIME_ERROR = 2,
  FLHIP_DECLINED = 3     /* only from the *_plan entry points: that kernel family does not take the geometry */
};

/* Storage type of activations.  Reductions and accumulators are always fp32.
 * Flashlight has no bf16 dtype (flashlight/fl/tensor/Types.h:17-30); FLHIP_BF16
 * is this library's private tag for bf16 storage with fp32 accumulate.
 * FLHIP_F16 is IEEE half storage, Flashlight's f16 (Types.h:17-30), which its cuDNN extension supports
 * (cudnn/CudnnAutogradExtension.cpp:27-36) and its oneDNN extension refuses
 * (onednn/OneDnnAutogradExtension.cpp:12-16).  Every entry point that takes FLHIP_BF16 takes FLHIP_F16 with
 * the same meaning (16-bit tensors where bf16 ones are, fp32 ones where fp32 ones are; results rounded once,
 * to nearest even, overflow to infinity); its tensors go through the kernels that widen their operands to
 * fp32, not through the bf16 matrix-core families. */
enum {
  FLHIP_F32 = 0,
  FLHIP_BF16 = 1,
  FLHIP_F16 = 2
};

/* fl::PoolingMode, same numeric values (flashlight/fl/common/Defines.h:53-64). */
enum {
  FLHIP_POOL_MAX = 0,
  FLHIP_POOL_AVG_INCLUDE_PADDING = 1,
  FLHIP_POOL_AVG_EXCLUDE_PADDING = 2
};

/* Which convolution pass a workspace query is for. */
enum {
  FLHIP_CONV_FWD = 0,
  FLHIP_CONV_BWD_DATA = 1,
  FLHIP_CONV_BWD_FILTER = 2
};

/* Convolution geometry.  x is [N,C,H,W], w is [K,C/groups,KH,KW], y is
 * [N,K,OH,OW] with OH = 1 + (H + 2*py - (1 + (KH-1)*dil_y)) / sy (integer
 * division), likewise OW (onednn/Conv2D.cpp:179-188).  Dilation uses
 * Flashlight's convention (1 = dense).  dtype = FLHIP_F32: every buffer fp32.
 * dtype = FLHIP_BF16 / FLHIP_F16: x, w, y, dy, dx are 16-bit; bias, dw, db stay fp32. */
typedef struct flhip_conv_desc {
  int32_t N, C, H, W;
  int32_t K, KH, KW;
  int32_t sy, sx;
  int32_t py, px;
  int32_t dil_y, dil_x;
  int32_t groups;
  int32_t dtype;
} flhip_conv_desc;

/* Pooling geometry.  x is [N,C,H,W]; y is [N,C,OH,OW], OH = 1 + (H + 2*py - wy)/sy
 * (onednn/Pool2D.cpp:100-102).  Padding is symmetric and must be smaller than the
 * window.  dtype tags x, y, dy and dx. */
typedef struct flhip_pool_desc {
  int32_t N, C, H, W;
  int32_t wy, wx;
  int32_t sy, sx;
  int32_t py, px;
  int32_t mode;
  int32_t dtype;
} flhip_pool_desc;

/* Batch-norm view, as the oneDNN extension derives it from the feature axes
 * (onednn/BatchNorm.cpp:40-71): element (o, c, i) lives at (o*C + c)*inner + i.
 * Spatial mode (axes do not include dim 0): outer = product of dims after the
 * last feature axis, inner = product of dims before the first.  Per-activation
 * mode (axes start at dim 0): inner = 1, outer = elements / C.
 * dtype tags x, y, dy, dx; gamma, beta, statistics and their gradients are fp32. */
typedef struct flhip_bn_desc {
  int64_t outer;
  int64_t C;
  int64_t inner;
  int32_t dtype;
} flhip_bn_desc;

const char* flhip_last_error(void);

/* Library version, and the gfx architecture the kernels were compiled for.  The version a caller was
 * compiled against is FLHIP_VERSION; descriptor structs only ever grow at the end, and a caller must
 * refuse to run when flhip_version() / 100 differs from FLHIP_VERSION / 100 (a layout change).
 * 200: flhip_rnn_desc gained dropout, seed_lo, seed_hi; flhip_bn_workspace_bytes never returns less
 * than 32 bytes per feature.  202: the *_plan entry points and FLHIP_DECLINED.  203: FLHIP_F16.  204: flhip_act_fwd / _bwd, flhip_glu_fwd / _bwd,
 * flhip_dropout, flhip_rownorm, flhip_weightnorm_fwd / _bwd, flhip_pad_fwd / _bwd, flhip_sgd_many, flhip_adam_many.  205: flhip_prelu_fwd / _bwd, FLHIP_ACT_LEAKY, FLHIP_ACT_THRESHOLD. */
#define FLHIP_VERSION 206
int flhip_version(void);
const char* flhip_arch(void);

/* Measurement / debugging switches.  Each is read once from the environment variable
 * FLHIP_<name> when the library first needs it; afterwards only this call changes it
 * (value NULL restores the default; the FLHIP_ prefix on `name` is optional).  Not to be
 * called while another thread is inside the library.  Results stay within the stated
 * tolerances under every setting; the switches only choose between kernels.
 *   CONV_ALGO = direct | gather | tapped | convert | auto    CONV_SKIP = bf16,gemm1x1,slab,tapped,strip,first,wgrad128,pwdma,wd32,tap1d,cells,tap2d
 *   PW_PT = 2 | 4 | 8    PW16_PF = 0 | 1 | 2 | 4 | 8    CONV_STACK = 0 | 1 | 2 | 4 | 8    BN_ALGO = split | resident | auto
 *   SLAB_WAVES = 0 | 4 | 8
 *   PW16_NO_TAPS, TAPPED_NO_REORDER, MATMUL_VALU, MATMUL_FP32_CORES, RNN_UNFUSED, TAP2D_ALL = 1 | 0
 *   MATMUL_PLANES = 0..7 (bit m: the fp32 product of form m - 0: A B, 1: A^T B, 2: A B^T - takes a matrix as one
 *                   image's plane whatever its shape; 0: never; unset: by shape)
 * Unknown names or values return FLHIP_INVALID_ARGUMENT.  The nearest thing in the
 * reference is the kernel-choice options object of its cuDNN extension
 * (createBenchmarkOptions, flashlight/fl/autograd/tensor/backend/cudnn/CudnnAutogradExtension.h:25). */
int flhip_set_option(const char* name, const char* value);

/* Output extents of the geometries above; return FLHIP_INVALID_ARGUMENT when the
 * geometry is not valid (non-positive sizes, window larger than padded input…). */
int flhip_conv2d_out_dims(const flhip_conv_desc* d, int32_t* OH, int32_t* OW);
int flhip_pool2d_out_dims(const flhip_pool_desc* d, int32_t* OH, int32_t* OW);

/* Scratch a convolution pass uses (0 is possible).  The filter gradient needs it (partial
 * results of the sliced contraction); forward and backward-data run without it too, but
 * with it the kernels for strided / long windows read weights reordered per tap, and
 * strided windows in bf16 storage run on the bf16 matrix cores over a gathered copy of
 * the input's lattice points (1x1, all passes) or of its taps (up to 9, backward passes), and
 * windows of one row (KH = 1, 2 to 32 taps, column stride 1 or 2: the 21 x 1 windows of a speech
 * stack; bf16 and fp32) run on kernels that read a channels-last copy of the source and weights
 * reordered into the order of the matrix instruction's fragments. */
size_t flhip_conv2d_workspace_bytes(const flhip_conv_desc* d, int pass);

/* AutogradExtension::conv2d (AutogradExtension.h:58-69; oneDNN peer
 * onednn/Conv2D.cpp:155-270): y = cross-correlation(x, w) + bias.  bias may be
 * NULL (the reference's "bias.elements() == 0"). */
int flhip_conv2d_fwd(const flhip_conv_desc* d, const void* x, const void* w,
                     const float* bias, void* y, void* ws, size_t ws_bytes,
                     void* stream);

/* AutogradExtension::conv2dBackwardData (AutogradExtension.h:110-122; oneDNN
 * peer onednn/Conv2D.cpp:272-375): dx = d(loss)/d(x) from dy and w. */
int flhip_conv2d_bwd_data(const flhip_conv_desc* d, const void* dy,
                          const void* w, void* dx, void* ws, size_t ws_bytes,
                          void* stream);

/* dx = addend + conv2dBackwardData(dy, w): the backward-data pass of the conv2d closure
 * (flashlight/fl/autograd/Functions.cpp:1362-1389) followed by Variable::addGrad
 * (Variable.cpp:185-218) when the input already holds a gradient (the shortcut's, at the head
 * of a residual block), in one pass over dx where the kernel allows it (bf16 1x1 stride 1;
 * everything else runs the two operations).  Both terms are rounded to the storage type
 * before the sum, so the result equals the two separate calls bit for bit.  addend has dx's
 * shape and type; dx must not alias it. */
int flhip_conv2d_bwd_data_add(const flhip_conv_desc* d, const void* dy, const void* w,
                              const void* addend, void* dx, void* ws, size_t ws_bytes,
                              void* stream);

/* AutogradExtension::conv2dBackwardFilterBias (AutogradExtension.h:124-138;
 * oneDNN peer onednn/Conv2D.cpp:377-507): dw (fp32, weight shape) and, when db
 * is not NULL, db[k] = sum of dy over n, oh, ow (fp32).  dw may be NULL to get
 * the bias gradient alone. */
int flhip_conv2d_bwd_filter(const flhip_conv_desc* d, const void* x,
                            const void* dy, float* dw, float* db, void* ws,
                            size_t ws_bytes, void* stream);

/* The payload that the conv2d closure hands from the forward call to the backward calls
 * (flashlight/fl/autograd/Functions.cpp:1341-1363: `payload`, captured by gradFunc; the oneDNN peer leaves it
 * empty).  With bf16 storage the forward pass of a strided layer first gathers the input points that its
 * windows touch (a 1x1 stride-2 layer: a quarter of the input; a 3x3 stride-2 layer: one copy per tap, 9/4 of
 * it) and runs as a 1x1 stride-1 layer over that copy; the filter gradient needs the same copy.  Likewise,
 * in bf16 and fp32, the forward pass of a window of one row first writes the input with its channels last,
 * and the filter gradient of such a window (6 to 23 taps) reads the same rows.
 * flhip_conv2d_gathered_bytes(d) > 0 says that flhip_conv2d_fwd leaves this copy in the first that many bytes
 * of its workspace.  A caller that keeps those bytes unchanged until the backward pass hands them to
 * flhip_conv2d_bwd_filter_gathered in place of x and saves the second gather (the six strided layers of
 * ResNet-50 at batch 64: 178 us of a step).  Results are bit-identical to flhip_conv2d_bwd_filter's.
 * ws as for flhip_conv2d_bwd_filter.  FLHIP_INVALID_ARGUMENT where flhip_conv2d_gathered_bytes(d) is 0. */
size_t flhip_conv2d_gathered_bytes(const flhip_conv_desc* d);
int flhip_conv2d_bwd_filter_gathered(const flhip_conv_desc* d, const void* gathered,
                                     const void* dy, float* dw, float* db, void* ws,
                                     size_t ws_bytes, void* stream);

/* The same filter / bias gradient for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It
 * has no counterpart in the reference.  The partial results of the sliced contraction
 * go to a buffer of FLHIP_STATIC_SCRATCH_BYTES that is part of the library's code
 * object (each GPU the library runs on holds one copy until the process ends); no
 * hipMalloc / hipFree or other allocating call is made.  Geometries whose
 * flhip_conv2d_workspace_bytes(d, FLHIP_CONV_BWD_FILTER) exceeds that size are refused
 * with FLHIP_INVALID_ARGUMENT.  Results are bit-identical to flhip_conv2d_bwd_filter.
 * The device of `stream` must be the current device.  All calls on one GPU share the
 * buffer: calls that overlap in time on one GPU (different streams, or threads) race. */
#define FLHIP_STATIC_SCRATCH_BYTES (40u << 20)
int flhip_conv2d_bwd_filter_static(const flhip_conv_desc* d, const void* x,
                                   const void* dy, float* dw, float* db,
                                   void* stream);

/* Kernel choice for the two backward passes, measured instead of ruled: what the reference reaches through
 * AutogradExtension::createBenchmarkOptions (AutogradExtension.h:53-55; the options object its caller closure makes
 * per pass, flashlight/fl/autograd/Functions.cpp:1372-1388, and that cudnn/Conv2D.cpp:467-520, 654-707 audits).
 * A pass has flhip_conv2d_plan_count(pass) kernel families ("plans", numbered in the order of the default rule;
 * flhip_conv2d_plan_name gives a family's description, NULL for numbers outside the list).  The *_plan entry
 * points are flhip_conv2d_bwd_data / flhip_conv2d_bwd_filter with one more argument: plan < 0 runs the default
 * rule (identical to the entry points above), plan >= 0 runs that family alone, whatever the rules and
 * switches say, or returns FLHIP_DECLINED without launching anything when the family does not take the
 * geometry or storage type, or when the workspace is too small for it.  Workspace as for the entry points above (their
 * size covers every plan; the stacked-plane plan of backward-data on planes of at most 32 x 32 positions).  Every
 * plan meets the stated tolerances; results of different plans differ in summation order only. */
int flhip_conv2d_plan_count(int pass);
const char* flhip_conv2d_plan_name(int pass, int plan);
int flhip_conv2d_bwd_data_plan(const flhip_conv_desc* d, const void* dy, const void* w, void* dx, void* ws,
                               size_t ws_bytes, int plan, void* stream);
int flhip_conv2d_bwd_filter_plan(const flhip_conv_desc* d, const void* x, const void* dy, float* dw, float* db,
                                 void* ws, size_t ws_bytes, int plan, void* stream);

/* AutogradExtension::pool2d (AutogradExtension.h:71-80; oneDNN peer
 * onednn/Pool2D.cpp:78-176).  For FLHIP_POOL_MAX with argmax != NULL the kernel
 * also writes one byte per output: the window-relative index kh*wx + kw of the
 * first maximum in (kh outer, kw inner) scan order under strict '>', padded
 * positions skipped — the workspace the reference keeps in its payload
 * (onednn/Pool2D.cpp:150-161).  Needs wy*wx <= 256 when argmax is requested. */
int flhip_pool2d_fwd(const flhip_pool_desc* d, const void* x, void* y,
                     uint8_t* argmax, void* stream);

/* AutogradExtension::pool2dBackward (AutogradExtension.h:141-152; oneDNN peer
 * onednn/Pool2D.cpp:178-247).  MAX needs the argmax bytes of the forward call;
 * the average modes ignore it.  Every element of dx is written (no pre-zeroing). */
int flhip_pool2d_bwd(const flhip_pool_desc* d, const void* dy,
                     const uint8_t* argmax, void* dx, void* stream);

/* Scratch for the batch-norm passes below (partial sums). */
size_t flhip_bn_workspace_bytes(const flhip_bn_desc* d);

/* AutogradExtension::batchnorm with train = true (AutogradExtension.h:82-94;
 * oneDNN peer onednn/BatchNorm.cpp:88-200; cuDNN peer cudnn/BatchNorm.cpp:145-162).
 * Batch mean and biased variance per feature; y = gamma*(x-mean)*invstd + beta.
 * gamma/beta NULL = ones/zeros.  save_mean/save_invstd (fp32[C]) receive the
 * batch mean and 1/sqrt(var+eps) for the backward pass.  When run_mean/run_var
 * are not NULL they are updated in place: momentum == 0 stores the batch mean
 * and biased variance (what the oneDNN extension does, BatchNorm.cpp:154-157);
 * momentum != 0 blends r = (1-momentum)*r + momentum*batch with the unbiased
 * batch variance (cuDNN semantics). */
int flhip_bn_fwd_train(const flhip_bn_desc* d, const void* x,
                       const float* gamma, const float* beta, void* y,
                       float* save_mean, float* save_invstd, float* run_mean,
                       float* run_var, double momentum, double eps, void* ws,
                       size_t ws_bytes, void* stream);

/* AutogradExtension::batchnorm with train = false (use_global_stats,
 * onednn/BatchNorm.cpp:171-175): y = gamma*(x-run_mean)/sqrt(run_var+eps)+beta. */
int flhip_bn_fwd_infer(const flhip_bn_desc* d, const void* x,
                       const float* gamma, const float* beta,
                       const float* run_mean, const float* run_var, double eps,
                       void* y, void* stream);

/* AutogradExtension::batchnormBackward (AutogradExtension.h:155-164; oneDNN peer
 * onednn/BatchNorm.cpp:202-279): dbeta = sum dy, dgamma = sum dy*xhat,
 * dx = gamma*invstd*(dy - dbeta/M - xhat*dgamma/M), M = outer*inner. */
int flhip_bn_bwd(const flhip_bn_desc* d, const void* x, const void* dy,
                 const float* gamma, const float* save_mean,
                 const float* save_invstd, void* dx, float* dgamma,
                 float* dbeta, void* ws, size_t ws_bytes, void* stream);

/* Batch norm fused with what follows it in a ResNet block (ConvBnAct and the block tails of
 * flashlight/pkg/vision/models/Resnet.cpp:27-46, 95-140: BatchNorm -> ReLU, and BatchNorm ->
 * "+ shortcut" -> ReLU): y = relu(bn(x) + residual) in the one pass that writes y, instead of
 * three trips through memory.  residual may be NULL; relu == 0 leaves the ReLU out.  Every
 * other argument as flhip_bn_fwd_train.  Segment mode only (inner > 1): per-activation
 * views return FLHIP_INVALID_ARGUMENT.  The reference has no fused counterpart; it composes
 * AutogradExtension::batchnorm, operator+ and fl::relu (Functions.cpp:111-121, 329-338). */
int flhip_bn_act_fwd_train(const flhip_bn_desc* d, const void* x, const float* gamma,
                           const float* beta, const void* residual, int relu, void* y,
                           float* save_mean, float* save_invstd, float* run_mean,
                           float* run_var, double momentum, double eps, void* ws,
                           size_t ws_bytes, void* stream);

/* Its backward: dz = dy where y > 0, else 0 (y = the forward result, the ReLU's mask); then
 * the batch-norm backward of flhip_bn_bwd on dz.  dresidual (may be NULL) receives dz, the
 * gradient of the residual input.  For a forward call with relu == 0 use flhip_bn_bwd. */
int flhip_bn_act_bwd(const flhip_bn_desc* d, const void* x, const void* dy, const void* y,
                     const float* gamma, const float* save_mean, const float* save_invstd,
                     void* dx, void* dresidual, float* dgamma, float* dbeta, void* ws,
                     size_t ws_bytes, void* stream);

/* The same pair with the ReLU's mask kept as bits instead of read back from y: the forward
 * call also writes one byte per 4 consecutive elements (bit e of byte i set where
 * y[4*i + e] > 0), the backward call reads those bytes in place of y: a quarter of a byte
 * per element instead of the 2 or 4 bytes of the forward result.  Rows must hold a
 * multiple of 4 elements (inner % 4 == 0): flhip_bn_act_mask_bytes gives the size of the
 * mask buffer, 0 where this form does not apply.  The gradients equal flhip_bn_act_bwd's bit
 * for bit.  Like the pair above, no counterpart in the reference. */
size_t flhip_bn_act_mask_bytes(const flhip_bn_desc* d);
int flhip_bn_act_fwd_train_mask(const flhip_bn_desc* d, const void* x, const float* gamma,
                                const float* beta, const void* residual, int relu, void* y,
                                void* mask, float* save_mean, float* save_invstd,
                                float* run_mean, float* run_var, double momentum, double eps,
                                void* ws, size_t ws_bytes, void* stream);
int flhip_bn_act_bwd_mask(const flhip_bn_desc* d, const void* x, const void* dy, const void* mask,
                          const float* gamma, const float* save_mean, const float* save_invstd,
                          void* dx, void* dresidual, float* dgamma, float* dbeta, void* ws,
                          size_t ws_bytes, void* stream);

/* Storage conversion among FLHIP_F32, FLHIP_BF16 and FLHIP_F16 (round to nearest even; between the
 * two 16-bit types through the fp32 value) of n elements; same dtype = copy.  Serves the casts the caller closures make around
 * the extension (Tensor::astype in flashlight/fl/autograd/Functions.cpp:1558-1561
 * and FL_ADJUST_INPUT_TYPE, flashlight/fl/autograd/Functions.h:57-82). */
int flhip_convert(const void* src, int src_dtype, void* dst, int dst_dtype,
                  size_t n, void* stream);
/* The same conversion of `count` tensors (src[i] -> dst[i], n[i] elements; host arrays of device
 * pointers) in one launch per 64 of them: the per-step casts of a network's fp32 master weights
 * to the storage type of its activations (the astype calls of Conv2D / Linear::forward,
 * flashlight/fl/nn/modules/Conv2D.cpp:157-176, Linear.cpp:60-72) are dozens of tensors of a few
 * kilobytes to megabytes, each a launch of its own otherwise. */
int flhip_convert_many(const void* const* src, void* const* dst, const size_t* n, int count,
                       int src_dtype, int dst_dtype, void* stream);
/* How flhip_convert_many cuts such a list into launches (at most 64 tensors and 2^31 - 1 pieces of 2048
 * elements each): returns the number of launches and, when launch_of is not null, the launch of
 * every tensor (-1 for empty ones); -1 for an argument flhip_convert_many would refuse.  Host code
 * only, no device call. */
int flhip_convert_many_launches(const size_t* n, int count, int* launch_of);

/* dst[i] = value for n elements of `dtype`: fl::full as the extension uses it for
 * default running statistics (onednn/BatchNorm.cpp:116-122), enqueued like every other
 * kernel (no host buffer, no synchronisation; safe under graph capture). */
int flhip_fill(void* dst, double value, size_t n, int dtype, void* stream);

/* fl::SGDOptimizer::step (flashlight/fl/optim/SGDOptimizer.cpp:38-68) over `count` parameter tensors of one dtype,
 * in place, one launch per 48 tensors: g = grad + weight_decay w; with momentum != 0, v = momentum v + g (stored) and
 * g = nesterov ? g + momentum v : v; w = w - lr g.  velocities may be NULL when momentum == 0. */
int flhip_sgd_many(void* const* params, const void* const* grads, void* const* velocities, const size_t* n,
                   int count, double lr, double momentum, double weight_decay, int nesterov, int dtype,
                   void* stream);

/* fl::AdamOptimizer::step (flashlight/fl/optim/AdamOptimizer.cpp:45-79), in place, one launch per 32 tensors:
 * w = w - weight_decay lr w; first = beta1 first + (1 - beta1) g; second = beta2 second + (1 - beta2) g g;
 * w = w - clr first / (sqrt(second) + epsilon), clr = lr sqrt(1 - beta2^step) / (1 - beta1^step); step counts from 1. */
int flhip_adam_many(void* const* params, const void* const* grads, void* const* first, void* const* second,
                    const size_t* n, int count, double lr, double beta1, double beta2, double epsilon,
                    double weight_decay, int64_t step, int dtype, void* stream);

/* out = a + b over n elements of `dtype` (out may alias a or b): the gradient
 * accumulation of Variable::addGrad (flashlight/fl/autograd/Variable.cpp:185-218). */
int flhip_add(const void* a, const void* b, void* out, size_t n, int dtype,
              void* stream);

/* ---- operations of the caller closures (flashlight/fl/autograd/Functions.cpp) ----
 * What a network of conv / pool / batch-norm layers needs besides the extension to
 * run one training step on device memory.  Matrices are column-major like
 * Flashlight tensors: element (r, c) of an R x C matrix is at r + c*R. */

/* fl::relu = max(x, 0) (Functions.cpp:329-338, 1787-1789) and its backward
 * dx = dy where x > 0, else 0. */
int flhip_relu_fwd(const void* x, void* y, size_t n, int dtype, void* stream);
int flhip_relu_bwd(const void* dy, const void* x, void* dx, size_t n, int dtype,
                   void* stream);

/* The other element-wise activations of fl::nn (flashlight/fl/nn/modules/Activations.cpp), one entry point:
 * y = f(x) over n elements, fp32 arithmetic, 16-bit storage rounded once.
 *   FLHIP_ACT_ELU      a = alpha: x >= 0 ? x : a (exp(x) - 1)                  (Activations.cpp:136-139)
 *   FLHIP_ACT_CLAMP    a = lo, b = hi: fl::clamp (Functions.cpp:465-475); ReLU6 = clamp(0, 6), HardTanh = clamp(-1, 1)
 *                      (Activations.cpp:60-62, 88-90)
 *   FLHIP_ACT_TANH     fl::tanh (Functions.cpp:454-463)      FLHIP_ACT_LOG      fl::log (:403-411)
 *   FLHIP_ACT_SWISH    a = beta: x * sigmoid(a x) (:498-500)  FLHIP_ACT_SIGMOID  fl::sigmoid (:488-496)
 *   FLHIP_ACT_SCALE    a x: a Variable times a number (the scales of fl::Residual, contrib/modules/Residual.cpp:69-73)
 *   FLHIP_ACT_LEAKY    a = slope: max(x, a x) (LeakyReLU, Activations.cpp:102-104); the gradient is fl::max's
 *                      (Functions.cpp:315-327): dy where x > a x, a dy elsewhere
 *   FLHIP_ACT_THRESHOLD  a = threshold: x where x >= a, else 0 (ThresholdReLU, Activations.cpp:151-154)
 * flhip_act_bwd: dx = dy * f'(x) from the gradient and the forward INPUT (clamp passes the gradient where
 * lo < x < hi, strictly, as the reference's mask on its result does).  y / dx may alias x / dy. */
#define FLHIP_ACT_ELU 0
#define FLHIP_ACT_CLAMP 1
#define FLHIP_ACT_TANH 2
#define FLHIP_ACT_LOG 3
#define FLHIP_ACT_SWISH 4
#define FLHIP_ACT_SIGMOID 5
#define FLHIP_ACT_SCALE 6
#define FLHIP_ACT_LEAKY 7
#define FLHIP_ACT_THRESHOLD 8
int flhip_act_fwd(int op, const void* x, void* y, size_t n, double a, double b, int dtype, void* stream);
int flhip_act_bwd(int op, const void* dy, const void* x, void* dx, size_t n, double a, double b, int dtype,
                  void* stream);

/* fl::gatedlinearunit (Functions.cpp:1567-1610) along a dimension whose two halves are contiguous blocks of m
 * elements per outer index (column-major tensor, halved dimension d: m = half the extent of d times the product of
 * the extents before it, outer = the product of the extents after it): y[o][k] = x[o][0][k] * sigmoid(x[o][1][k]);
 * backward dx[o][0][k] = sigmoid(x[o][1][k]) dy, dx[o][1][k] = x[o][0][k] s (1 - s) dy.  dx must not alias x. */
int flhip_glu_fwd(const void* x, void* y, int64_t outer, int64_t m, int dtype, void* stream);
int flhip_glu_bwd(const void* dy, const void* x, void* dx, int64_t outer, int64_t m, int dtype, void* stream);

/* fl::dropout (Functions.cpp:1777-1785): y = x * keep / (1 - p) with keep(i) a counter-based function of
 * (seed, i) - the reference draws fl::rand(...) > p, so masks differ from its generator's while rate and scaling
 * are the same.  The backward pass is the same call on the gradient with the same seed and p.  y may alias x. */
int flhip_dropout(const void* x, void* y, size_t n, double p, uint32_t seed_lo, uint32_t seed_hi, int dtype,
                  void* stream);

/* fl::WeightNorm (flashlight/fl/nn/modules/WeightNorm.cpp:45-72): w = v * g[r] / ||v_r||, one g per index r of the
 * kept dimension, the norm over all the others.  The tensor is a rows x cols matrix: rows_fast != 0 when the kept
 * dimension is the tensor's first (element (r, j) at r + j * rows: Linear weights, dim 0), 0 when it is the last
 * (element (r, j) at r * cols + j: Conv2D weights, dim 3) - the two the reference accepts.  g, n and dg have `rows`
 * elements of the tensor's dtype.  flhip_rownorm gives ||v_r|| (the initial g, :68-72).  Backward (the chain of the
 * reference's norm / division / tileAs / product): dv = (g / n) (dw - c v / n^2), dg[r] = c / n, c = sum_j dw v. */
int flhip_rownorm(const void* v, void* n, int64_t rows, int64_t cols, int rows_fast, int dtype, void* stream);
int flhip_weightnorm_fwd(const void* v, const void* g, void* w, int64_t rows, int64_t cols, int rows_fast,
                         int dtype, void* stream);
int flhip_weightnorm_bwd(const void* dw, const void* v, const void* g, void* dv, void* dg, int64_t rows,
                         int64_t cols, int rows_fast, int dtype, void* stream);

/* fl::padding (Functions.cpp:1751-1775) of a tensor with the four column-major extents dims[0..3] (pad with 1):
 * before[k] / after[k] elements of `value` in front of / behind dimension k.  flhip_pad_bwd copies the inner box of
 * the padded gradient back (dims, before, after as in the forward call).  Buffers must not overlap. */
int flhip_pad_fwd(const void* x, void* y, const int64_t* dims, const int32_t* before, const int32_t* after,
                  double value, int dtype, void* stream);
int flhip_pad_bwd(const void* dy, void* dx, const int64_t* dims, const int32_t* before, const int32_t* after,
                  int dtype, void* stream);

/* C (M x N) = op(A) (M x K) * op(B) (K x N), fp32 accumulate, one rounding to the element
 * type; trans_a: A is stored K x M, trans_b: B is stored N x K.  bias_rows (fp32[M], may be
 * NULL) is added to every column.  bf16 / f16 products of more than 128 columns run on the
 * 16-bit matrix instructions (option MATMUL_FP32_CORES: on the fp32 ones).  Serves fl::linear (Functions.cpp:1255-1309): forward
 * matmul(weight, input) + tile(bias), backward matmulTN(weight, gradOutput) and
 * matmulNT(gradOutput, input). */
int flhip_matmul(const void* A, const void* B, void* C, int32_t M, int32_t N,
                 int32_t K, int trans_a, int trans_b, const float* bias_rows,
                 int dtype, void* stream);
/* The same product with a workspace.  A * B^T with few tiles of C over a long contraction
 * (matmulNT(gradOutput, input), Functions.cpp:1297-1303, of a layer over many frames) leaves
 * most of the chip idle; with flhip_matmul_workspace_bytes(...) bytes at ws (0: this product
 * has no use for one) the contraction is cut into slices, one workgroup per tile and slice,
 * whose fp32 partial products are added in slice order (the result does not depend on
 * timing).  ws == NULL or fewer bytes: as flhip_matmul. */
size_t flhip_matmul_workspace_bytes(int32_t M, int32_t N, int32_t K, int trans_a, int trans_b, int dtype);
int flhip_matmul_ws(const void* A, const void* B, void* C, int32_t M, int32_t N,
                    int32_t K, int trans_a, int trans_b, const float* bias_rows,
                    int dtype, void* ws, size_t ws_bytes, void* stream);

/* out[r] (fp32) = sum over c of x[r, c] for a rows x cols matrix: the bias gradient
 * sumAs(gradOutput, bias) of fl::linear (Functions.cpp:1285-1289). */
int flhip_sum_columns(const void* x, float* out, int32_t rows, int32_t cols, int dtype,
                      void* stream);
/* The same sums with a workspace: few rows over many columns (a layer over many frames) are
 * few workgroups for flhip_sum_columns; with flhip_sum_columns_workspace_bytes(...) bytes at
 * ws (0: no use for one) the columns are cut into slices whose partial sums are added in
 * slice order.  ws == NULL or fewer bytes: as flhip_sum_columns. */
size_t flhip_sum_columns_workspace_bytes(int32_t rows, int32_t cols, int dtype);
int flhip_sum_columns_ws(const void* x, float* out, int32_t rows, int32_t cols, int dtype,
                         void* ws, size_t ws_bytes, void* stream);

/* fl::reorder (flashlight/fl/autograd/Functions.cpp:1010-1042) of a tensor with the four
 * column-major extents dims[0..3] (dims[0] fastest; pad with 1): dimension k of dst is
 * dimension perm[k] of src.  LayerNorm uses it when the axes it batches over are not
 * contiguous (flashlight/fl/nn/modules/LayerNorm.cpp:63-86, 98-108).  src and dst must not
 * overlap. */
int flhip_reorder(const void* src, void* dst, const int64_t* dims, const int32_t* perm,
                  int dtype, void* stream);

/* The affine part of fl::LayerNorm (flashlight/fl/nn/modules/LayerNorm.cpp:110-128),
 * tileAs(weight, input) * output + tileAs(bias, input), on a tensor viewed as
 * [outer][mid][inner] (inner fastest): y = w[m] * x + b[m] with one parameter element
 * per mid index, or a single element when scalar_params != 0.  w and b have the
 * tensor's dtype. */
int flhip_affine_fwd(const void* x, const void* w, const void* b, void* y, int64_t outer,
                     int64_t mid, int64_t inner, int scalar_params, int dtype,
                     void* stream);
/* Its backward: dx = w * dy (skipped when dx is NULL), dw[m] = sum of dy * x and
 * db[m] = sum of dy over the elements that share parameter m (fp32, either may be
 * NULL).  The sums are two-stage with a fixed order; the workspace holds the
 * partials and is needed only when dw or db is asked for. */
size_t flhip_affine_bwd_workspace_bytes(int64_t outer, int64_t mid, int64_t inner,
                                        int scalar_params);
int flhip_affine_bwd(const void* dy, const void* x, const void* w, void* dx, float* dw,
                     float* db, int64_t outer, int64_t mid, int64_t inner,
                     int scalar_params, int dtype, void* workspace,
                     size_t workspace_bytes, void* stream);

/* fl::embedding (Functions.cpp:1707-1749): y[:, i] = w[:, idx[i]] for n indices (s32 on the device) into a
 * dim x tokens table; an index outside [0, tokens) gives a column of zeros.  Backward (there a CSR matrix of ones
 * times the transposed deltas): dw[:, t] = the sum of dy[:, i] over idx[i] == t, added in the order of i in fp32 and
 * rounded once, zeros for tokens that do not occur; every column of dw is written. */
int flhip_embedding_fwd(const int32_t* idx, const void* w, void* y, int64_t n, int32_t dim, int32_t tokens, int dtype,
                        void* stream);
int flhip_embedding_bwd(const int32_t* idx, const void* dy, void* dw, int64_t n, int32_t dim, int32_t tokens, int dtype,
                        void* stream);

/* fl::PReLU (flashlight/fl/nn/modules/Activations.cpp:116-124): y = x where x >= 0, w[m] x elsewhere, the parameter
 * tiled along the tensor's first (fastest) dimension of extent d0 (m = element index % d0, `outer` = the product of
 * the other extents) or a single element (scalar_param != 0).  w has the tensor's dtype.  Backward (the chain of
 * the reference's mask, products and tileAs): dx = dy where x >= 0, w[m] dy elsewhere (skipped when dx is NULL);
 * dw[m] (fp32, may be NULL) = the sum of dy x over the elements with x < 0 that share m, two-stage in a fixed
 * order through the workspace. */
int flhip_prelu_fwd(const void* x, const void* w, void* y, int64_t outer, int64_t d0, int scalar_param, int dtype,
                    void* stream);
size_t flhip_prelu_bwd_workspace_bytes(int64_t outer, int64_t d0, int scalar_param);
int flhip_prelu_bwd(const void* dy, const void* x, const void* w, void* dx, float* dw, int64_t outer, int64_t d0,
                    int scalar_param, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* fl::logSoftmax over dimension 0 of a classes x cols matrix (Functions.cpp:1044-1070)
 * and its backward dx = dy - exp(y) * sum over classes of dy. */
int flhip_logsoftmax_fwd(const void* x, void* y, int32_t classes, int32_t cols,
                         int dtype, void* stream);
int flhip_logsoftmax_bwd(const void* dy, const void* y, void* dx, int32_t classes,
                         int32_t cols, int dtype, void* stream);

/* fl::categoricalCrossEntropy on log-probabilities logp (classes x cols) and int32
 * targets (Functions.cpp:1078-1154).  stats (fp32[4], device) receives: [0] the sum of
 * -logp[target, col] over counted columns (ReduceMode::SUM), [1] the number of counted
 * columns (target != ignore_index), [2] the number of columns whose target is outside
 * [0, classes) and not ignore_index (the reference throws std::invalid_argument for
 * those, :1100-1108: the host reads this entry), [3] = [0] / [1] (ReduceMode::MEAN).
 * per_column (fp32[cols], may be NULL) receives the unreduced values (ReduceMode::NONE).
 * Backward: dx[c, col] = -g where c == target[col] and the column counts, else 0, with
 * g = grad[col] (reduction 0 = NONE), grad[0] / stats[1] (1 = MEAN) or grad[0] (2 = SUM);
 * grad is fp32 on the device. */
int flhip_cce_fwd(const void* logp, const int32_t* target, float* stats,
                  float* per_column, int32_t classes, int32_t cols,
                  int32_t ignore_index, int dtype, void* stream);
int flhip_cce_bwd(const float* grad, const int32_t* target, const float* stats, void* dx,
                  int32_t classes, int32_t cols, int reduction, int32_t ignore_index,
                  int dtype, void* stream);

/* Plain device-to-device copy kernel of `bytes` bytes (multiple of 16).  Not part
 * of the operator interface: it is the known-size kernel that hardware byte
 * counters are calibrated against when measuring the kernels above. */
int flhip_copy_bytes(const void* src, void* dst, size_t bytes, void* stream);

/* ---- rnn / rnnBackward (flashlight/fl/autograd/tensor/AutogradExtension.h:96-106,
 * 167-179) with the semantics and the flat weight order of the cuDNN calls behind
 * CudnnAutogradExtension::rnn (backend/cudnn/RNN.cpp:62-375): per pseudo-layer
 * (layer-major, forward direction first) the input matrices of every gate
 * ([hidden][in], row-major) then the recurrent ones; after all matrices, per
 * pseudo-layer the input biases then the recurrent biases.  Gates: LSTM i, f, g, o;
 * GRU r, z, n.  mode: 0 ReLU, 1 tanh, 2 LSTM, 3 GRU (fl::RnnMode).  x is Flashlight
 * [input, batch, seq] (memory [seq][batch][input]), hx / cx / hy / cy
 * [hidden, batch, layers*dirs], y [hidden*dirs, batch, seq].  fp32 only.
 * dropout (RNN.cpp:83-90, training): the output sequence of every layer but the last is
 * multiplied by keep / (1 - dropout) before the next layer reads it; the states hy / cy are
 * not touched.  keep is a counter-based mask of (seed, layer, element index) - cuDNN draws
 * from a generator of its own, so WHICH elements fall is particular to this library; the
 * backward call must be given the descriptor of its forward call (same dropout and seed). */
typedef struct flhip_rnn_desc {
  int32_t input_size, hidden_size, num_layers, bidirectional, mode, seq_len, batch, dtype;
  float dropout;              /* 0 <= dropout < 1; 0 = none */
  uint32_t seed_lo, seed_hi;  /* of the dropout mask */
} flhip_rnn_desc;
/* number of weight elements (cudnnGetRNNParamsSize / element size); 0 for a bad descriptor */
size_t flhip_rnn_param_count(const flhip_rnn_desc* d);
/* the reserve buffer carries the forward pass's states and gate activations to the
 * backward pass (cuDNN's reserve space, RNN.cpp:154-160); the workspace is scratch */
size_t flhip_rnn_reserve_bytes(const flhip_rnn_desc* d);
size_t flhip_rnn_workspace_bytes(const flhip_rnn_desc* d);
/* hx, cx may be NULL (zero initial state); cy may be NULL */
int flhip_rnn_fwd(const flhip_rnn_desc* d, const void* x, const void* hx, const void* cx,
                  const void* w, void* y, void* hy, void* cy, void* reserve,
                  size_t reserve_bytes, void* workspace, size_t workspace_bytes, void* stream);
/* dy, dhy, dcy may be NULL (zero gradient, the closure's empty tensors,
 * Functions.cpp:1677-1699); dhx, dcx may be NULL; dw has flhip_rnn_param_count elements */
int flhip_rnn_bwd(const flhip_rnn_desc* d, const void* x, const void* w, const void* dy,
                  const void* dhy, const void* dcy, const void* reserve, size_t reserve_bytes,
                  void* dx, void* dhx, void* dcx, void* dw, void* workspace,
                  size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLHIP_H */
