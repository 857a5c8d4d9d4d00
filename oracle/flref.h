/*
 * flref — CPU restatement of the arithmetic behind Flashlight's oneDNN
 * AutogradExtension (conv2d, pool2d, batchnorm and their backward passes).
 *
 * TEST INFRASTRUCTURE ONLY.  This is the checker the HIP kernels are compared
 * with; nothing in the shipped library or its host layer calls it.
 *
 * The reference delegates the arithmetic to oneDNN (un-vendored, not pinned:
 * find_package(DNNL), flashlight/fl/tensor/backend/onednn/CMakeLists.txt:6), so
 * each function restates the published definition of the primitive the
 * reference requests, with the shapes, flags and quirks of the reference's own
 * call site (cited per function).  Layout is the reference's: row-major
 * N,C,H,W == Flashlight column-major [W,H,C,N].
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   conv fwd / bwd-data / bwd-filter+bias: brute-force definition in numpy on
 *     tiny cases, adjoint identities, 1x1-conv == GEMM, batching invariance, the
 *     shapes of the reference's own Jacobian tests, and PyTorch-CPU's library
 *     routines (oneDNN v3.7.1 inside) on seeded cases.
 *   pool fwd / bwd (max, avg include/exclude padding): brute force with ties on
 *     a 1/8 grid, sum(dx) == sum(dy), library routines.
 *   batchnorm train / infer / backward: the closed forms of the reference's
 *     tests (AutogradNormalizationTest.cpp:37-226), invariants sum(dx) == 0 and
 *     sum(dx*xhat) == 0, finite differences, library routines.
 *   caller closures (relu, matmul / linear, sum over columns, logSoftmax,
 *     categoricalCrossEntropy, the LayerNorm affine part): float64 numpy
 *     definitions and torch.nn.functional with its autograd.
 *   rnn / rnnBackward: torch.nn.RNN / LSTM / GRU in float64 (same gate formulas and
 *     weight order as cuDNN), forward and autograd, stacked and bidirectional, and
 *     the parameter counts of the reference's test (AutogradRnnTest.cpp:37-49).
 * Not pinned by anything the reference holds ("parity unpinned" there, fixed
 * here by the definition above and checked against oneDNN through PyTorch):
 * the max-pool tie order and the running-statistics update for momentum != 0.
 */
#ifndef FLREF_H
#define FLREF_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct flref_conv {
  int32_t N, C, H, W;
  int32_t K, KH, KW;
  int32_t sy, sx, py, px, dil_y, dil_x, groups;
} flref_conv;

typedef struct flref_pool {
  int32_t N, C, H, W;
  int32_t wy, wx, sy, sx, py, px;
  int32_t mode; /* 0 max, 1 avg include padding, 2 avg exclude padding */
} flref_pool;

int flref_conv_out(const flref_conv* d, int32_t* OH, int32_t* OW);
int flref_pool_out(const flref_pool* d, int32_t* OH, int32_t* OW);

/* onednn/Conv2D.cpp:155-270 */
void flref_conv2d_fwd(const flref_conv* d, const float* x, const float* w,
                      const float* bias, float* y);
/* onednn/Conv2D.cpp:272-375 */
void flref_conv2d_bwd_data(const flref_conv* d, const float* dy, const float* w,
                           float* dx);
/* onednn/Conv2D.cpp:377-507 */
void flref_conv2d_bwd_filter(const flref_conv* d, const float* x,
                             const float* dy, float* dw, float* db);

/* onednn/Pool2D.cpp:78-176.  argmax (may be NULL) gets kh*wx+kw per output. */
void flref_pool2d_fwd(const flref_pool* d, const float* x, float* y,
                      uint8_t* argmax);
/* onednn/Pool2D.cpp:178-247 */
void flref_pool2d_bwd(const flref_pool* d, const float* dy,
                      const uint8_t* argmax, float* dx);

/* onednn/BatchNorm.cpp:88-200; element (o,c,i) at (o*C + c)*inner + i. */
void flref_bn_fwd_train(int64_t outer, int64_t C, int64_t inner, const float* x,
                        const float* gamma, const float* beta, double eps,
                        float* y, float* mean, float* var);
void flref_bn_fwd_infer(int64_t outer, int64_t C, int64_t inner, const float* x,
                        const float* gamma, const float* beta,
                        const float* mean, const float* var, double eps,
                        float* y);
/* onednn/BatchNorm.cpp:202-279 */
void flref_bn_bwd(int64_t outer, int64_t C, int64_t inner, const float* x,
                  const float* dy, const float* gamma, const float* mean,
                  const float* var, double eps, float* dx, float* dgamma,
                  float* dbeta);

/* Running-statistics update.  momentum == 0: overwrite with batch mean and
 * biased variance (onednn/BatchNorm.cpp:154-157 binds the running buffers as the
 * primitive's mean/variance outputs).  Otherwise r = (1-m)*r + m*batch with the
 * unbiased variance var*M/(M-1) (cudnnBatchNormalizationForwardTraining, called
 * at cudnn/BatchNorm.cpp:145-162). */
void flref_bn_running_update(int64_t C, int64_t M, const float* mean,
                             const float* var, double momentum, float* run_mean,
                             float* run_var);

/* ---- caller closures (flashlight/fl/autograd/Functions.cpp); column-major matrices:
 * element (r, c) of an R x C matrix at r + c*R ---- */
/* max(x, 0) and its mask backward (:329-338, 1787-1789) */
void flref_relu_fwd(int64_t n, const float* x, float* y);
void flref_relu_bwd(int64_t n, const float* dy, const float* x, float* dx);
/* element-wise activations of nn/modules/Activations.cpp: op 0 ELU(a), 1 clamp(a, b), 2 tanh, 3 log, 4 swish(a),
 * 5 sigmoid; the backward takes the forward input */
void flref_act_fwd(int op, int64_t n, const float* x, double a, double b, float* y);
void flref_act_bwd(int op, int64_t n, const float* dy, const float* x, double a, double b, float* dx);
/* gatedlinearunit (:1567-1610): halves are contiguous blocks of m elements per outer index */
void flref_glu_fwd(int64_t outer, int64_t m, const float* x, float* y);
void flref_glu_bwd(int64_t outer, int64_t m, const float* dy, const float* x, float* dx);
void flref_embedding_fwd(int64_t n, int64_t dim, int64_t tokens, const int32_t* idx, const float* w, float* y);
void flref_embedding_bwd(int64_t n, int64_t dim, int64_t tokens, const int32_t* idx, const float* dy, float* dw);
void flref_prelu_fwd(int64_t n, int64_t d0, int64_t size, const float* x, const float* w, float* y);
void flref_prelu_bwd(int64_t n, int64_t d0, int64_t size, const float* dy, const float* x, const float* w, float* dx,
                     float* dw);
/* dropout (:1777-1785) with the counter-based mask of flref_dropout_keep */
void flref_dropout(int64_t n, const float* x, double p, uint32_t seed_lo, uint32_t seed_hi, float* y);
/* WeightNorm (nn/modules/WeightNorm.cpp:45-72) over a rows x cols view (rows_fast: element (r, j) at r + j*rows,
 * else r*cols + j): row norms, w = v g / ||v||, and the gradients of v and g */
void flref_rownorm(int64_t rows, int64_t cols, int rows_fast, const float* v, float* n);
void flref_weightnorm_fwd(int64_t rows, int64_t cols, int rows_fast, const float* v, const float* g, float* w);
void flref_weightnorm_bwd(int64_t rows, int64_t cols, int rows_fast, const float* dw, const float* v, const float* g,
                          float* dv, float* dg);
/* fl::padding (:1751-1775) over four column-major extents and the slice back */
void flref_pad_fwd(const int64_t* dims, const int32_t* before, const int32_t* after, double value, const float* x, float* y);
void flref_pad_bwd(const int64_t* dims, const int32_t* before, const int32_t* after, const float* dy, float* dx);
/* SGD with weight decay, momentum and Nesterov momentum (optim/SGDOptimizer.cpp:38-68), in place; v may be NULL when mu == 0 */
void flref_sgd(int64_t n, float* w, const float* g, float* v, double lr, double mu, double wd, int nesterov);
/* Adam with decoupled weight decay (optim/AdamOptimizer.cpp:45-79), in place; step counts from 1 */
void flref_adam(int64_t n, float* w, const float* g, float* m, float* v, double lr, double b1, double b2, double eps,
                double wd, int64_t step);
/* C (M x N) = op(A) op(B) + bias[m]; ta: A stored K x M, tb: B stored N x K; double
 * accumulate.  fl::linear (:1255-1309) = (W, X), backward (W^T, dY) and (dY, X^T). */
void flref_matmul(int M, int N, int K, int ta, int tb, const float* A, const float* B,
                  const float* bias, float* C);
/* out[r] = sum_c x[r, c] (sumAs(gradOutput, bias), :1285-1289) */
void flref_sum_columns(int rows, int cols, const float* x, float* out);

/* Affine part of fl::LayerNorm (flashlight/fl/nn/modules/LayerNorm.cpp:110-128):
 * y = tileAs(w) * x + tileAs(b) on a tensor viewed as [outer][mid][inner]; the
 * parameters have `mid` elements, or one when scalar != 0.  Backward: dx = w * dy,
 * dw = sum of dy * x and db = sum of dy over the tiled dimensions (the gradients of
 * the broadcast multiply and add). */
void flref_affine_fwd(int64_t outer, int64_t mid, int64_t inner, int scalar, const float* x,
                      const float* w, const float* b, float* y);
void flref_affine_bwd(int64_t outer, int64_t mid, int64_t inner, int scalar, const float* dy,
                      const float* x, const float* w, float* dx, float* dw, float* db);
/* logSoftmax over dimension 0 of a classes x cols matrix (:1044-1070) */
void flref_logsoftmax_fwd(int classes, int cols, const float* x, float* y);
void flref_logsoftmax_bwd(int classes, int cols, const float* dy, const float* y, float* dx);
/* categoricalCrossEntropy (:1078-1154): returns the number of targets outside
 * [0, classes) that are not ignore; loss[0] = SUM, loss[1] = MEAN, count = counted columns */
int flref_cce_fwd(int classes, int cols, const float* logp, const int32_t* target, int ignore,
                  float* per_column, float* loss, float* count);
void flref_cce_bwd(int classes, int cols, const float* grad, const int32_t* target, int ignore,
                   int reduction, float count, float* dx);

/* ---- AutogradExtension::rnn / rnnBackward (flashlight/fl/autograd/tensor/
 * AutogradExtension.h:96-106,167-179) with the semantics of the cuDNN extension
 * (backend/cudnn/RNN.cpp:62-375; the oneDNN one has no backward, onednn/RNN.cpp:558-573):
 * x [T][B][input] (Flashlight [input, B, T]), hx / hy / cx / cy [layers*dirs][B][hidden],
 * y [T][B][dirs*hidden] (forward direction first), all row-major.  The weights are one
 * flat vector in cuDNN's order: per pseudo-layer (layer-major, forward direction first)
 * the input matrices of every gate ([hidden][in], row-major) then the recurrent ones
 * ([hidden][hidden]); after all matrices, per pseudo-layer the input biases then the
 * recurrent biases.  Gates: LSTM i, f, g, o; GRU r, z, n with
 * n = tanh(W_n x + b_Wn + r * (R_n h + b_Rn)), h' = (1 - z) * n + z * h.
 * mode: 0 ReLU, 1 tanh, 2 LSTM, 3 GRU (flashlight/fl/common/Defines.h:62-67).
 * dropout > 0 (training, flashlight/fl/autograd/tensor/backend/cudnn/RNN.cpp:83-90): the
 * output sequence of every layer but the last is multiplied, element by element, by
 * keep / (1 - dropout) before the next layer reads it; keep = flref_dropout_keep().  cuDNN
 * draws its mask from a generator of its own: which elements are dropped is a property
 * of this restatement (parity unpinned against the reference), where the mask is applied
 * and how it scales follows cuDNN's documented behaviour and is checked against torch. */
typedef struct flref_rnn {
  int32_t input_size, hidden, layers, bidirectional, mode, T, B;
  float dropout;
  uint32_t seed_lo, seed_hi;
} flref_rnn;
/* 1 if element `index` of the output of layer `layer` is kept */
int flref_dropout_keep(uint32_t seed_lo, uint32_t seed_hi, uint32_t layer, uint32_t index, float dropout);
int64_t flref_rnn_param_count(const flref_rnn* d);
/* hx, cx may be NULL (zeros); cy may be NULL */
void flref_rnn_fwd(const flref_rnn* d, const float* x, const float* hx, const float* cx,
                   const float* w, float* y, float* hy, float* cy);
/* dy, dhy, dcy may be NULL (zeros); dhx, dcx may be NULL (not wanted) */
void flref_rnn_bwd(const flref_rnn* d, const float* x, const float* hx, const float* cx,
                   const float* w, const float* dy, const float* dhy, const float* dcy,
                   float* dx, float* dhx, float* dcx, float* dw);

#ifdef __cplusplus
}
#endif
#endif
