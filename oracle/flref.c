/* CPU restatement used as the parity checker; see flref.h for what it is and
 * how it is pinned.  Convolution and batch-norm accumulate in double (the
 * checker should sit closer to the exact result than either fp32
 * implementation); pooling is done in fp32 in the reference's scan order so
 * that the comparison with the device kernels can be bit-exact. */
#include "flref.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

static inline int div_floor(int a, int b) {
  int q = a / b;
  if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
  return q;
}
static inline int div_ceil(int a, int b) { return -div_floor(-a, b); }
static inline int imax(int a, int b) { return a > b ? a : b; }
static inline int imin(int a, int b) { return a < b ? a : b; }

/* Output extent, onednn/Conv2D.cpp:179-188 (integer division). */
int flref_conv_out(const flref_conv* d, int32_t* OH, int32_t* OW) {
  int eh = 1 + (d->KH - 1) * d->dil_y, ew = 1 + (d->KW - 1) * d->dil_x;
  if (d->H + 2 * d->py < eh || d->W + 2 * d->px < ew) return 1;
  *OH = 1 + (d->H + 2 * d->py - eh) / d->sy;
  *OW = 1 + (d->W + 2 * d->px - ew) / d->sx;
  return 0;
}

/* Output extent, onednn/Pool2D.cpp:100-102. */
int flref_pool_out(const flref_pool* d, int32_t* OH, int32_t* OW) {
  if (d->H + 2 * d->py < d->wy || d->W + 2 * d->px < d->wx) return 1;
  *OH = 1 + (d->H + 2 * d->py - d->wy) / d->sy;
  *OW = 1 + (d->W + 2 * d->px - d->wx) / d->sx;
  return 0;
}

/* Range of ow for which iw = ow*s - p + off lies in [0, W). */
static inline void valid_range(int O, int W, int s, int p, int off, int* lo,
                               int* hi) {
  *lo = imax(0, div_ceil(p - off, s));
  *hi = imin(O - 1, div_floor(W - 1 + p - off, s));
}

/* Cross-correlation with zero padding, groups as the goihw view of
 * [kx,ky,Cin/g,Cout] (onednn/Conv2D.cpp:69-93), Flashlight dilation d = oneDNN
 * d-1 (:103-105), optional bias (:189). */
void flref_conv2d_fwd(const flref_conv* d, const float* x, const float* w,
                      const float* bias, float* y) {
  int32_t OH, OW;
  if (flref_conv_out(d, &OH, &OW)) return;
  const int Cg = d->C / d->groups, Kg = d->K / d->groups;
  const long planes = (long)d->N * d->K;
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * OH * OW);
#pragma omp for schedule(static)
    for (long pk = 0; pk < planes; ++pk) {
      const int n = (int)(pk / d->K), k = (int)(pk % d->K), g = k / Kg;
      const double b = bias ? (double)bias[k] : 0.0;
      for (int i = 0; i < OH * OW; ++i) acc[i] = b;
      for (int c = 0; c < Cg; ++c) {
        const float* xp = x + ((long)n * d->C + g * Cg + c) * d->H * d->W;
        for (int kh = 0; kh < d->KH; ++kh) {
          int oh0, oh1;
          valid_range(OH, d->H, d->sy, d->py, kh * d->dil_y, &oh0, &oh1);
          for (int kw = 0; kw < d->KW; ++kw) {
            const double wv = w[(((long)k * Cg + c) * d->KH + kh) * d->KW + kw];
            int ow0, ow1;
            valid_range(OW, d->W, d->sx, d->px, kw * d->dil_x, &ow0, &ow1);
            for (int oh = oh0; oh <= oh1; ++oh) {
              const int ih = oh * d->sy - d->py + kh * d->dil_y;
              const float* xr = xp + (long)ih * d->W - d->px + kw * d->dil_x;
              double* ar = acc + (long)oh * OW;
              for (int ow = ow0; ow <= ow1; ++ow)
                ar[ow] += wv * (double)xr[ow * d->sx];
            }
          }
        }
      }
      float* yp = y + pk * OH * OW;
      for (int i = 0; i < OH * OW; ++i) yp[i] = (float)acc[i];
    }
    free(acc);
  }
}

/* dx[n,c,ih,iw] = sum over (k,kh,kw,oh,ow) hitting (ih,iw) of dy*w; result has
 * the input's shape (onednn/Conv2D.cpp:285). */
void flref_conv2d_bwd_data(const flref_conv* d, const float* dy, const float* w,
                           float* dx) {
  int32_t OH, OW;
  if (flref_conv_out(d, &OH, &OW)) return;
  const int Cg = d->C / d->groups, Kg = d->K / d->groups;
  const long planes = (long)d->N * d->C;
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * d->H * d->W);
#pragma omp for schedule(static)
    for (long pc = 0; pc < planes; ++pc) {
      const int n = (int)(pc / d->C), ci = (int)(pc % d->C), g = ci / Cg,
                c = ci % Cg;
      for (int i = 0; i < d->H * d->W; ++i) acc[i] = 0.0;
      for (int kk = 0; kk < Kg; ++kk) {
        const int k = g * Kg + kk;
        const float* dyp = dy + ((long)n * d->K + k) * OH * OW;
        for (int kh = 0; kh < d->KH; ++kh) {
          int oh0, oh1;
          valid_range(OH, d->H, d->sy, d->py, kh * d->dil_y, &oh0, &oh1);
          for (int kw = 0; kw < d->KW; ++kw) {
            const double wv = w[(((long)k * Cg + c) * d->KH + kh) * d->KW + kw];
            int ow0, ow1;
            valid_range(OW, d->W, d->sx, d->px, kw * d->dil_x, &ow0, &ow1);
            for (int oh = oh0; oh <= oh1; ++oh) {
              const int ih = oh * d->sy - d->py + kh * d->dil_y;
              double* ar = acc + (long)ih * d->W - d->px + kw * d->dil_x;
              const float* dr = dyp + (long)oh * OW;
              for (int ow = ow0; ow <= ow1; ++ow)
                ar[ow * d->sx] += wv * (double)dr[ow];
            }
          }
        }
      }
      float* dxp = dx + pc * d->H * d->W;
      for (int i = 0; i < d->H * d->W; ++i) dxp[i] = (float)acc[i];
    }
    free(acc);
  }
}

/* dw[k,c,kh,kw] = sum over (n,oh,ow) of dy*x; db[k] = sum over (n,oh,ow) of dy,
 * produced by the same primitive when a bias exists (onednn/Conv2D.cpp:411-415,
 * 486-489).  dw or db may be NULL. */
void flref_conv2d_bwd_filter(const flref_conv* d, const float* x,
                             const float* dy, float* dw, float* db) {
  int32_t OH, OW;
  if (flref_conv_out(d, &OH, &OW)) return;
  const int Cg = d->C / d->groups, Kg = d->K / d->groups;
  if (dw) {
    const long rows = (long)d->K * Cg;
#pragma omp parallel for schedule(static)
    for (long kc = 0; kc < rows; ++kc) {
      const int k = (int)(kc / Cg), c = (int)(kc % Cg), g = k / Kg;
      for (int kh = 0; kh < d->KH; ++kh) {
        int oh0, oh1;
        valid_range(OH, d->H, d->sy, d->py, kh * d->dil_y, &oh0, &oh1);
        for (int kw = 0; kw < d->KW; ++kw) {
          int ow0, ow1;
          valid_range(OW, d->W, d->sx, d->px, kw * d->dil_x, &ow0, &ow1);
          double s = 0.0;
          for (int n = 0; n < d->N; ++n) {
            const float* xp = x + ((long)n * d->C + g * Cg + c) * d->H * d->W;
            const float* dyp = dy + ((long)n * d->K + k) * OH * OW;
            for (int oh = oh0; oh <= oh1; ++oh) {
              const int ih = oh * d->sy - d->py + kh * d->dil_y;
              const float* xr = xp + (long)ih * d->W - d->px + kw * d->dil_x;
              const float* dr = dyp + (long)oh * OW;
              double r = 0.0;
              for (int ow = ow0; ow <= ow1; ++ow)
                r += (double)dr[ow] * (double)xr[ow * d->sx];
              s += r;
            }
          }
          dw[(kc * d->KH + kh) * d->KW + kw] = (float)s;
        }
      }
    }
  }
  if (db) {
#pragma omp parallel for schedule(static)
    for (int k = 0; k < d->K; ++k) {
      double s = 0.0;
      for (int n = 0; n < d->N; ++n) {
        const float* dyp = dy + ((long)n * d->K + k) * OH * OW;
        double r = 0.0;
        for (int i = 0; i < OH * OW; ++i) r += (double)dyp[i];
        s += r;
      }
      db[k] = (float)s;
    }
  }
}

/* Max: running maximum starts at the lowest float; a window element replaces it
 * only under strict '>', scanning kh outer / kw inner and skipping padded
 * positions, so ties keep the first maximum (oneDNN's reference pooling, the
 * primitive requested at onednn/Pool2D.cpp:125-135).  Averages: fp32 sum in scan
 * order divided by wy*wx (include padding) or by the in-bounds count (exclude),
 * modes mapped as in DnnlUtils.cpp:145-156. */
void flref_pool2d_fwd(const flref_pool* d, const float* x, float* y,
                      uint8_t* argmax) {
  int32_t OH, OW;
  if (flref_pool_out(d, &OH, &OW)) return;
  const long planes = (long)d->N * d->C;
#pragma omp parallel for schedule(static)
  for (long p = 0; p < planes; ++p) {
    const float* xp = x + p * d->H * d->W;
    float* yp = y + p * OH * OW;
    uint8_t* ap = argmax ? argmax + p * OH * OW : 0;
    for (int oh = 0; oh < OH; ++oh)
      for (int ow = 0; ow < OW; ++ow) {
        float best = -FLT_MAX, sum = 0.f;
        int idx = 0, cnt = 0;
        for (int kh = 0; kh < d->wy; ++kh) {
          const int ih = oh * d->sy - d->py + kh;
          if (ih < 0 || ih >= d->H) continue;
          for (int kw = 0; kw < d->wx; ++kw) {
            const int iw = ow * d->sx - d->px + kw;
            if (iw < 0 || iw >= d->W) continue;
            const float v = xp[(long)ih * d->W + iw];
            if (v > best) {
              best = v;
              idx = kh * d->wx + kw;
            }
            sum += v;
            ++cnt;
          }
        }
        if (d->mode == 0) {
          yp[oh * OW + ow] = best;
          if (ap) ap[oh * OW + ow] = (uint8_t)idx;
        } else if (d->mode == 1) {
          yp[oh * OW + ow] = sum / (float)(d->wy * d->wx);
        } else {
          yp[oh * OW + ow] = sum / (float)cnt;
        }
      }
  }
}

/* dx starts at zero; windows are visited in ascending (oh, ow) and add into dx
 * in fp32: max routes dy to the recorded argmax, averages spread dy/divisor
 * over the in-bounds window positions (onednn/Pool2D.cpp:178-247). */
void flref_pool2d_bwd(const flref_pool* d, const float* dy,
                      const uint8_t* argmax, float* dx) {
  int32_t OH, OW;
  if (flref_pool_out(d, &OH, &OW)) return;
  const long planes = (long)d->N * d->C;
#pragma omp parallel for schedule(static)
  for (long p = 0; p < planes; ++p) {
    float* dxp = dx + p * d->H * d->W;
    const float* dyp = dy + p * OH * OW;
    const uint8_t* ap = argmax ? argmax + p * OH * OW : 0;
    for (long i = 0; i < (long)d->H * d->W; ++i) dxp[i] = 0.f;
    for (int oh = 0; oh < OH; ++oh)
      for (int ow = 0; ow < OW; ++ow) {
        const float g = dyp[oh * OW + ow];
        if (d->mode == 0) {
          const int idx = ap[oh * OW + ow];
          const int ih = oh * d->sy - d->py + idx / d->wx;
          const int iw = ow * d->sx - d->px + idx % d->wx;
          dxp[(long)ih * d->W + iw] += g;
          continue;
        }
        int cnt = d->wy * d->wx;
        if (d->mode == 2) {
          const int h0 = imax(oh * d->sy - d->py, 0),
                    h1 = imin(oh * d->sy - d->py + d->wy, d->H);
          const int w0 = imax(ow * d->sx - d->px, 0),
                    w1 = imin(ow * d->sx - d->px + d->wx, d->W);
          cnt = (h1 - h0) * (w1 - w0);
        }
        const float q = g / (float)cnt;
        for (int kh = 0; kh < d->wy; ++kh) {
          const int ih = oh * d->sy - d->py + kh;
          if (ih < 0 || ih >= d->H) continue;
          for (int kw = 0; kw < d->wx; ++kw) {
            const int iw = ow * d->sx - d->px + kw;
            if (iw < 0 || iw >= d->W) continue;
            dxp[(long)ih * d->W + iw] += q;
          }
        }
      }
  }
}

/* Train mode: per-feature mean and biased (population) variance over (outer,
 * inner); y = gamma*(x-mean)/sqrt(var+eps)+beta with use_scale|use_shift
 * (onednn/BatchNorm.cpp:171-175).  gamma/beta NULL = ones/zeros (:136-139). */
void flref_bn_fwd_train(int64_t outer, int64_t C, int64_t inner, const float* x,
                        const float* gamma, const float* beta, double eps,
                        float* y, float* mean, float* var) {
  const double M = (double)outer * (double)inner;
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < C; ++c) {
    double s = 0.0;
    for (int64_t o = 0; o < outer; ++o) {
      const float* xp = x + (o * C + c) * inner;
      double r = 0.0;
      for (int64_t i = 0; i < inner; ++i) r += xp[i];
      s += r;
    }
    const double mu = s / M;
    double v = 0.0;
    for (int64_t o = 0; o < outer; ++o) {
      const float* xp = x + (o * C + c) * inner;
      double r = 0.0;
      for (int64_t i = 0; i < inner; ++i) {
        const double t = xp[i] - mu;
        r += t * t;
      }
      v += r;
    }
    v /= M;
    const double is = 1.0 / sqrt(v + eps);
    const double g = gamma ? gamma[c] : 1.0, b = beta ? beta[c] : 0.0;
    for (int64_t o = 0; o < outer; ++o) {
      const float* xp = x + (o * C + c) * inner;
      float* yp = y + (o * C + c) * inner;
      for (int64_t i = 0; i < inner; ++i)
        yp[i] = (float)(g * (xp[i] - mu) * is + b);
    }
    if (mean) mean[c] = (float)mu;
    if (var) var[c] = (float)v;
  }
}

/* Inference: use_global_stats (onednn/BatchNorm.cpp:171-175). */
void flref_bn_fwd_infer(int64_t outer, int64_t C, int64_t inner, const float* x,
                        const float* gamma, const float* beta,
                        const float* mean, const float* var, double eps,
                        float* y) {
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < C; ++c) {
    const double is = 1.0 / sqrt((double)var[c] + eps), mu = mean[c];
    const double g = gamma ? gamma[c] : 1.0, b = beta ? beta[c] : 0.0;
    for (int64_t o = 0; o < outer; ++o) {
      const float* xp = x + (o * C + c) * inner;
      float* yp = y + (o * C + c) * inner;
      for (int64_t i = 0; i < inner; ++i)
        yp[i] = (float)(g * (xp[i] - mu) * is + b);
    }
  }
}

/* prop_kind::backward with use_scale|use_shift (onednn/BatchNorm.cpp:249-259):
 * dbeta = sum dy, dgamma = sum dy*xhat,
 * dx = gamma*invstd*(dy - dbeta/M - xhat*dgamma/M). */
void flref_bn_bwd(int64_t outer, int64_t C, int64_t inner, const float* x,
                  const float* dy, const float* gamma, const float* mean,
                  const float* var, double eps, float* dx, float* dgamma,
                  float* dbeta) {
  const double M = (double)outer * (double)inner;
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < C; ++c) {
    const double mu = mean[c], is = 1.0 / sqrt((double)var[c] + eps);
    const double g = gamma ? gamma[c] : 1.0;
    double sb = 0.0, sg = 0.0;
    for (int64_t o = 0; o < outer; ++o) {
      const float* xp = x + (o * C + c) * inner;
      const float* dp = dy + (o * C + c) * inner;
      double rb = 0.0, rg = 0.0;
      for (int64_t i = 0; i < inner; ++i) {
        rb += dp[i];
        rg += (double)dp[i] * ((xp[i] - mu) * is);
      }
      sb += rb;
      sg += rg;
    }
    for (int64_t o = 0; o < outer; ++o) {
      const float* xp = x + (o * C + c) * inner;
      const float* dp = dy + (o * C + c) * inner;
      float* op = dx + (o * C + c) * inner;
      for (int64_t i = 0; i < inner; ++i) {
        const double xh = (xp[i] - mu) * is;
        op[i] = (float)(g * is * (dp[i] - sb / M - xh * sg / M));
      }
    }
    if (dgamma) dgamma[c] = (float)sg;
    if (dbeta) dbeta[c] = (float)sb;
  }
}

void flref_bn_running_update(int64_t C, int64_t M, const float* mean,
                             const float* var, double momentum, float* run_mean,
                             float* run_var) {
  for (int64_t c = 0; c < C; ++c) {
    if (momentum == 0.0) {
      run_mean[c] = mean[c];
      run_var[c] = var[c];
    } else {
      const double unb =
          M > 1 ? (double)var[c] * (double)M / (double)(M - 1) : var[c];
      run_mean[c] =
          (float)((1.0 - momentum) * run_mean[c] + momentum * mean[c]);
      run_var[c] = (float)((1.0 - momentum) * run_var[c] + momentum * unb);
    }
  }
}

/* ---- caller closures (flashlight/fl/autograd/Functions.cpp) ---------------------- */

/* fl::maximum(x, 0) (:329-338): NaN > 0 is false, so NaN maps to 0 as in the mask */
void flref_relu_fwd(int64_t n, const float* x, float* y) {
  for (int64_t i = 0; i < n; ++i) y[i] = x[i] > 0.f ? x[i] : 0.f;
}

/* mask = (x > 0) (:333-335) */
void flref_relu_bwd(int64_t n, const float* dy, const float* x, float* dx) {
  for (int64_t i = 0; i < n; ++i) dx[i] = x[i] > 0.f ? dy[i] : 0.f;
}

/* The element-wise activations of nn/modules/Activations.cpp, in double, rounded once.  op as FLHIP_ACT_*:
 * 0 ELU (a = alpha; :136-139 there), 1 clamp(a, b) (Functions.cpp:465-475), 2 tanh (:454-463), 3 log (:403-411),
 * 4 swish (a = beta; :498-500), 5 sigmoid (:488-496), 6 a x, 7 LeakyReLU max(x, a x) (:102-104 there, with
 * fl::max's gradient mask x > a x, Functions.cpp:315-327), 8 ThresholdReLU x * (x >= a) (:151-154). */
static double act_sigmoid(double v) { return 1.0 / (1.0 + exp(-v)); }
void flref_act_fwd(int op, int64_t n, const float* x, double a, double b, float* y) {
  for (int64_t i = 0; i < n; ++i) {
    const double v = x[i];
    double r;
    switch (op) {
      case 0: r = v >= 0.0 ? v : a * (exp(v) - 1.0); break;
      case 1: r = v < a ? a : v > b ? b : v; break;
      case 2: r = tanh(v); break;
      case 3: r = log(v); break;
      case 4: r = v * act_sigmoid(a * v); break;
      case 6: r = a * v; break;
      case 7: r = v > a * v ? v : a * v; break;
      case 8: r = v >= a ? v : 0.0; break;
      default: r = act_sigmoid(v); break;
    }
    y[i] = (float)r;
  }
}
/* gradients of the same: the reference's closures (ELU and swish: the chain of their element-wise pieces) */
void flref_act_bwd(int op, int64_t n, const float* dy, const float* x, double a, double b, float* dx) {
  for (int64_t i = 0; i < n; ++i) {
    const double v = x[i], g = dy[i];
    double r;
    switch (op) {
      case 0: r = v >= 0.0 ? g : g * a * exp(v); break;
      case 1: r = (v > a && v < b) ? g : 0.0; break;          /* (result > lo) && (result < hi), :471 */
      case 2: { const double t = tanh(v); r = (1.0 - t * t) * g; break; }
      case 3: r = g / v; break;
      case 4: { const double sg = act_sigmoid(a * v); r = g * (sg + v * a * sg * (1.0 - sg)); break; }
      case 6: r = a * g; break;
      case 7: r = v > a * v ? g : a * g; break;
      case 8: r = v >= a ? g : 0.0; break;
      default: { const double sg = act_sigmoid(v); r = g * sg * (1.0 - sg); break; }
    }
    dx[i] = (float)r;
  }
}

/* fl::gatedlinearunit (Functions.cpp:1567-1610) with the halves as contiguous blocks of m elements per outer index */
void flref_glu_fwd(int64_t outer, int64_t m, const float* x, float* y) {
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t k = 0; k < m; ++k)
      y[o * m + k] = (float)((double)x[2 * o * m + k] * act_sigmoid(x[(2 * o + 1) * m + k]));
}
void flref_glu_bwd(int64_t outer, int64_t m, const float* dy, const float* x, float* dx) {
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t k = 0; k < m; ++k) {
      const double a = x[2 * o * m + k], sg = act_sigmoid(x[(2 * o + 1) * m + k]), g = dy[o * m + k];
      dx[2 * o * m + k] = (float)(sg * g);                          /* :1598 */
      dx[(2 * o + 1) * m + k] = (float)(a * sg * (1.0 - sg) * g);   /* :1599-1600 */
    }
}

/* fl::PReLU (nn/modules/Activations.cpp:121-124): (input * mask) + (input * !mask * tileAs(w, input)) with mask =
 * input >= 0; the parameter has `size` elements tiled along the first dimension (extent d0, size divides d0).
 * Backward by the chain rule of those operators: dx = dy mask + dy !mask w, dw = sumAs(dy input !mask, w). */
void flref_prelu_fwd(int64_t n, int64_t d0, int64_t size, const float* x, const float* w, float* y) {
  for (int64_t i = 0; i < n; ++i) {
    const double mask = x[i] >= 0.f ? 1.0 : 0.0;
    y[i] = (float)((double)x[i] * mask + (double)x[i] * (1.0 - mask) * (double)w[(i % d0) % size]);
  }
}
void flref_prelu_bwd(int64_t n, int64_t d0, int64_t size, const float* dy, const float* x, const float* w, float* dx,
                     float* dw) {
  double* acc = (double*)calloc((size_t)size, sizeof(double));
  for (int64_t i = 0; i < n; ++i) {
    const double mask = x[i] >= 0.f ? 1.0 : 0.0;
    const int64_t m = (i % d0) % size;
    dx[i] = (float)((double)dy[i] * mask + (double)dy[i] * (1.0 - mask) * (double)w[m]);
    acc[m] += (double)dy[i] * (double)x[i] * (1.0 - mask);
  }
  for (int64_t m = 0; m < size; ++m) dw[m] = (float)acc[m];
  free(acc);
}

/* fl::embedding (Functions.cpp:1707-1749): y[:, i] = w[:, idx[i]] (column-major: dim rows per token); the gradient,
 * there a CSR matrix of ones times the transposed deltas, is dw[:, t] = the sum of dy[:, i] over idx[i] == t, in
 * double.  Indices outside [0, tokens) give a zero column and no gradient. */
void flref_embedding_fwd(int64_t n, int64_t dim, int64_t tokens, const int32_t* idx, const float* w, float* y) {
  for (int64_t i = 0; i < n; ++i)
    for (int64_t d = 0; d < dim; ++d)
      y[i * dim + d] = (idx[i] >= 0 && idx[i] < tokens) ? w[(int64_t)idx[i] * dim + d] : 0.f;
}
void flref_embedding_bwd(int64_t n, int64_t dim, int64_t tokens, const int32_t* idx, const float* dy, float* dw) {
  double* acc = (double*)calloc((size_t)(dim * tokens), sizeof(double));
  for (int64_t i = 0; i < n; ++i) {
    if (idx[i] < 0 || idx[i] >= tokens) continue;
    for (int64_t d = 0; d < dim; ++d) acc[(int64_t)idx[i] * dim + d] += (double)dy[i * dim + d];
  }
  for (int64_t k = 0; k < dim * tokens; ++k) dw[k] = (float)acc[k];
  free(acc);
}

/* fl::dropout (Functions.cpp:1777-1785) with the counter-based mask below in the place of fl::rand(...) > p */
int flref_dropout_keep(uint32_t seed_lo, uint32_t seed_hi, uint32_t layer, uint32_t index, float dropout);
void flref_dropout(int64_t n, const float* x, double p, uint32_t seed_lo, uint32_t seed_hi, float* y) {
  const float scale = (float)(1.0 / (1.0 - p));
  for (int64_t i = 0; i < n; ++i)
    y[i] = flref_dropout_keep(seed_lo, seed_hi, (uint32_t)((uint64_t)i >> 32), (uint32_t)i, (float)p) ? x[i] * scale : 0.f;
}

/* WeightNorm (nn/modules/WeightNorm.cpp:45-72): w = v g[r] / ||v_r|| over a rows x cols view, element (r, j) at
 * r + j*rows (rows_fast) or r*cols + j; in double */
static size_t wn_at(int64_t r, int64_t j, int64_t rows, int64_t cols, int rows_fast) {
  return rows_fast ? (size_t)r + (size_t)j * (size_t)rows : (size_t)r * (size_t)cols + (size_t)j;
}
void flref_rownorm(int64_t rows, int64_t cols, int rows_fast, const float* v, float* n) {
  for (int64_t r = 0; r < rows; ++r) {
    double s2 = 0.0;
    for (int64_t j = 0; j < cols; ++j) { const double x = v[wn_at(r, j, rows, cols, rows_fast)]; s2 += x * x; }
    n[r] = (float)sqrt(s2);
  }
}
void flref_weightnorm_fwd(int64_t rows, int64_t cols, int rows_fast, const float* v, const float* g, float* w) {
  for (int64_t r = 0; r < rows; ++r) {
    double s2 = 0.0;
    for (int64_t j = 0; j < cols; ++j) { const double x = v[wn_at(r, j, rows, cols, rows_fast)]; s2 += x * x; }
    const double scale = (double)g[r] / sqrt(s2);
    for (int64_t j = 0; j < cols; ++j) {
      const size_t e = wn_at(r, j, rows, cols, rows_fast);
      w[e] = (float)(v[e] * scale);
    }
  }
}
/* w = v s, s = g / n: dv = s dw + (dL/ds)(ds/dn)(dn/dv) = s (dw - c v / n^2), dg = c / n, c = sum dw v */
void flref_weightnorm_bwd(int64_t rows, int64_t cols, int rows_fast, const float* dw, const float* v, const float* g,
                          float* dv, float* dg) {
  for (int64_t r = 0; r < rows; ++r) {
    double s2 = 0.0, c = 0.0;
    for (int64_t j = 0; j < cols; ++j) {
      const size_t e = wn_at(r, j, rows, cols, rows_fast);
      s2 += (double)v[e] * v[e];
      c += (double)dw[e] * v[e];
    }
    const double n = sqrt(s2), scale = (double)g[r] / n;
    for (int64_t j = 0; j < cols; ++j) {
      const size_t e = wn_at(r, j, rows, cols, rows_fast);
      dv[e] = (float)(scale * ((double)dw[e] - c * v[e] / s2));
    }
    dg[r] = (float)(c / n);
  }
}

/* fl::padding (Functions.cpp:1751-1775), four column-major extents */
void flref_pad_fwd(const int64_t* dims, const int32_t* before, const int32_t* after, double value, const float* x, float* y) {
  int64_t od[4];
  for (int k = 0; k < 4; ++k) od[k] = dims[k] + before[k] + after[k];
  for (int64_t d = 0; d < od[3]; ++d)
    for (int64_t c = 0; c < od[2]; ++c)
      for (int64_t b = 0; b < od[1]; ++b)
        for (int64_t a = 0; a < od[0]; ++a) {
          const int64_t q[4] = {a - before[0], b - before[1], c - before[2], d - before[3]};
          int in = 1;
          for (int k = 0; k < 4; ++k) in = in && q[k] >= 0 && q[k] < dims[k];
          y[a + od[0] * (b + od[1] * (c + od[2] * d))] =
              in ? x[q[0] + dims[0] * (q[1] + dims[1] * (q[2] + dims[2] * q[3]))] : (float)value;
        }
}
void flref_pad_bwd(const int64_t* dims, const int32_t* before, const int32_t* after, const float* dy, float* dx) {
  int64_t od[4];
  for (int k = 0; k < 4; ++k) od[k] = dims[k] + before[k] + after[k];
  for (int64_t d = 0; d < dims[3]; ++d)
    for (int64_t c = 0; c < dims[2]; ++c)
      for (int64_t b = 0; b < dims[1]; ++b)
        for (int64_t a = 0; a < dims[0]; ++a)
          dx[a + dims[0] * (b + dims[1] * (c + dims[2] * d))] =
              dy[(a + before[0]) + od[0] * ((b + before[1]) + od[1] * ((c + before[2]) + od[2] * (d + before[3])))];
}

/* fl::SGDOptimizer::step (flashlight/fl/optim/SGDOptimizer.cpp:38-68) on one tensor, in place, in double with the
 * stored values rounded to float */
void flref_sgd(int64_t n, float* w, const float* g, float* v, double lr, double mu, double wd, int nesterov) {
  for (int64_t i = 0; i < n; ++i) {
    double gi = g[i];
    if (wd != 0.0) gi = gi + wd * w[i];
    if (mu != 0.0) {
      v[i] = (float)(mu * v[i] + gi);
      gi = nesterov ? gi + (double)v[i] * mu : (double)v[i];
    }
    w[i] = (float)((double)w[i] - lr * gi);
  }
}

/* fl::AdamOptimizer::step (optim/AdamOptimizer.cpp:45-79) on one tensor, in place; the corrected rate in float as there */
void flref_adam(int64_t n, float* w, const float* g, float* m, float* v, double lr, double b1, double b2, double eps,
                double wd, int64_t step) {
  const float cb1 = 1.f - powf((float)b1, (float)step), cb2 = 1.f - powf((float)b2, (float)step);
  const double clr = (float)lr * sqrtf(cb2) / cb1;
  for (int64_t i = 0; i < n; ++i) {
    double wi = w[i];
    const double gi = g[i];
    if (wd != 0.0) wi = wi - wd * lr * wi;
    m[i] = (float)(b1 * m[i] + (1.0 - b1) * gi);
    v[i] = (float)(b2 * v[i] + (1.0 - b2) * gi * gi);
    w[i] = (float)(wi - clr * m[i] / (sqrt((double)v[i]) + eps));
  }
}

/* fl::matmul / matmulTN / matmulNT as used by fl::linear (:1264-1265, 1292-1301) */
void flref_matmul(int M, int N, int K, int ta, int tb, const float* A, const float* B,
                  const float* bias, float* C) {
#pragma omp parallel for
  for (int n = 0; n < N; ++n)
    for (int m = 0; m < M; ++m) {
      double s = 0.0;
      for (int k = 0; k < K; ++k) {
        const double a = ta ? A[(size_t)k + (size_t)m * K] : A[(size_t)m + (size_t)k * M];
        const double b = tb ? B[(size_t)n + (size_t)k * N] : B[(size_t)k + (size_t)n * K];
        s += a * b;
      }
      C[(size_t)m + (size_t)n * M] = (float)(s + (bias ? (double)bias[m] : 0.0));
    }
}

void flref_sum_columns(int rows, int cols, const float* x, float* out) {
  for (int r = 0; r < rows; ++r) {
    double s = 0.0;
    for (int c = 0; c < cols; ++c) s += x[(size_t)r + (size_t)c * rows];
    out[r] = (float)s;
  }
}

/* LayerNorm.cpp:110-128: the parameter element of (o, m, i) is m, or 0 when scalar */
void flref_affine_fwd(int64_t outer, int64_t mid, int64_t inner, int scalar, const float* x,
                      const float* w, const float* b, float* y) {
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t m = 0; m < mid; ++m)
      for (int64_t i = 0; i < inner; ++i) {
        const int64_t e = (o * mid + m) * inner + i, pm = scalar ? 0 : m;
        y[e] = (float)((double)w[pm] * x[e] + b[pm]);
      }
}

void flref_affine_bwd(int64_t outer, int64_t mid, int64_t inner, int scalar, const float* dy,
                      const float* x, const float* w, float* dx, float* dw, float* db) {
  const int64_t np = scalar ? 1 : mid;
  double* acc = (double*)calloc((size_t)np * 2, sizeof(double));
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t m = 0; m < mid; ++m)
      for (int64_t i = 0; i < inner; ++i) {
        const int64_t e = (o * mid + m) * inner + i, pm = scalar ? 0 : m;
        if (dx) dx[e] = w[pm] * dy[e];
        acc[2 * pm] += (double)dy[e] * x[e];
        acc[2 * pm + 1] += dy[e];
      }
  for (int64_t m = 0; m < np; ++m) {
    if (dw) dw[m] = (float)acc[2 * m];
    if (db) db[m] = (float)acc[2 * m + 1];
  }
  free(acc);
}

/* x - (log(sum(exp(x - max))) + max) per column (:1046-1056) */
void flref_logsoftmax_fwd(int classes, int cols, const float* x, float* y) {
  for (int c = 0; c < cols; ++c) {
    const float* xc = x + (size_t)c * classes;
    double mx = xc[0];
    for (int k = 1; k < classes; ++k) mx = xc[k] > mx ? xc[k] : mx;
    double s = 0.0;
    for (int k = 0; k < classes; ++k) s += exp((double)xc[k] - mx);
    const double lse = log(s) + mx;
    for (int k = 0; k < classes; ++k) y[(size_t)c * classes + k] = (float)((double)xc[k] - lse);
  }
}

/* gradOutput - exp(result) * sum(gradOutput) (:1061-1066) */
void flref_logsoftmax_bwd(int classes, int cols, const float* dy, const float* y, float* dx) {
  for (int c = 0; c < cols; ++c) {
    const size_t o = (size_t)c * classes;
    double s = 0.0;
    for (int k = 0; k < classes; ++k) s += dy[o + k];
    for (int k = 0; k < classes; ++k) dx[o + k] = (float)((double)dy[o + k] - exp((double)y[o + k]) * s);
  }
}

/* -x[target] per column, ignored columns 0; MEAN divides by the counted columns
 * (:1112-1126) */
int flref_cce_fwd(int classes, int cols, const float* logp, const int32_t* target, int ignore,
                  float* per_column, float* loss, float* count) {
  int bad = 0;
  double s = 0.0, n = 0.0;
  for (int c = 0; c < cols; ++c) {
    const int t = target[c];
    double v = 0.0;
    if (t == ignore) {
    } else if (t < 0 || t >= classes) {
      ++bad;
    } else {
      v = -(double)logp[(size_t)c * classes + t];
      n += 1.0;
    }
    if (per_column) per_column[c] = (float)v;
    s += v;
  }
  loss[0] = (float)s;
  loss[1] = (float)(s / n);
  *count = (float)n;
  return bad;
}

/* tile(grad) * mask with mask = -(class == target), ignored columns 0 (:1135-1150) */
void flref_cce_bwd(int classes, int cols, const float* grad, const int32_t* target, int ignore,
                   int reduction, float count, float* dx) {
  for (int c = 0; c < cols; ++c) {
    const int t = target[c];
    const double g = reduction == 0 ? grad[c] : reduction == 1 ? (double)grad[0] / count : grad[0];
    for (int k = 0; k < classes; ++k)
      dx[(size_t)c * classes + k] = (t != ignore && k == t) ? (float)(-g) : 0.f;
  }
}


/* ---- rnn / rnnBackward ------------------------------------------------------------- */
static int rnn_gates(int mode) { return mode == 2 ? 4 : mode == 3 ? 3 : 1; }

int64_t flref_rnn_param_count(const flref_rnn* d) {
  const int64_t G = rnn_gates(d->mode), H = d->hidden, D = d->bidirectional ? 2 : 1;
  int64_t n = 0;
  for (int l = 0; l < d->layers; ++l) {
    const int64_t in = l == 0 ? d->input_size : D * H;
    n += D * (G * H * (in + H) + 2 * G * H);
  }
  return n;
}

/* offsets of pseudo-layer pl inside the flat weight vector */
static void rnn_offsets(const flref_rnn* d, int pl, int64_t* W, int64_t* R, int64_t* bW, int64_t* bR) {
  const int64_t G = rnn_gates(d->mode), H = d->hidden, D = d->bidirectional ? 2 : 1;
  int64_t off = 0, mats = 0;
  for (int p = 0; p < d->layers * D; ++p) {
    const int64_t in = p / D == 0 ? d->input_size : D * H;
    if (p == pl) {
      *W = off;
      *R = off + G * H * in;
    }
    off += G * H * (in + H);
  }
  mats = off;
  *bW = mats + (int64_t)pl * 2 * G * H;
  *bR = *bW + G * H;
}

static double sigm(double v) { return 1.0 / (1.0 + exp(-v)); }

/* Everything one pseudo-layer keeps for the way back, in step order s (time t = s for
 * the forward direction, T-1-s for the backward one). */
typedef struct rnn_tape {
  double* hprev; /* [T+1][B][H]: state before step s; entry T = final state */
  double* cprev; /* LSTM, same shape */
  double* gate;  /* [T][G][B][H] activations */
  double* rn;    /* GRU: R_n h + b_Rn, [T][B][H] */
} rnn_tape;

static void rnn_layer_fwd(const flref_rnn* d, int pl, const double* in, int64_t inl, const float* w,
                          const float* hx, const float* cx, double* out, rnn_tape* tp) {
  const int G = rnn_gates(d->mode), H = d->hidden, D = d->bidirectional ? 2 : 1, T = d->T, B = d->B;
  const int dir = pl % D;
  int64_t oW = 0, oR = 0, obW = 0, obR = 0;
  rnn_offsets(d, pl, &oW, &oR, &obW, &obR);
  const size_t BH = (size_t)B * H;
  for (size_t i = 0; i < BH; ++i) {
    tp->hprev[i] = hx ? hx[(size_t)pl * BH + i] : 0.0;
    if (tp->cprev) tp->cprev[i] = cx ? cx[(size_t)pl * BH + i] : 0.0;
  }
  double* a = (double*)malloc(sizeof(double) * G * H);
  double* r = (double*)malloc(sizeof(double) * G * H);
  for (int s = 0; s < T; ++s) {
    const int t = dir ? T - 1 - s : s;
    const double* hp = tp->hprev + (size_t)s * BH;
    double* hn = tp->hprev + (size_t)(s + 1) * BH;
    for (int b = 0; b < B; ++b) {
      const double* xin = in + ((size_t)t * B + b) * inl;
      for (int q = 0; q < G * H; ++q) {
        double sa = w[obW + q], sr = w[obR + q];
        for (int64_t i = 0; i < inl; ++i) sa += (double)w[oW + (int64_t)q * inl + i] * xin[i];
        for (int j = 0; j < H; ++j) sr += (double)w[oR + (int64_t)q * H + j] * hp[(size_t)b * H + j];
        a[q] = sa;
        r[q] = sr;
      }
      for (int h = 0; h < H; ++h) {
        double* gt = tp->gate + (size_t)s * G * BH + (size_t)b * H + h; /* + g*BH */
        double hv;
        if (d->mode == 0 || d->mode == 1) {
          const double pre = a[h] + r[h];
          hv = d->mode == 0 ? (pre > 0 ? pre : 0.0) : tanh(pre);
          gt[0] = hv;
        } else if (d->mode == 2) {
          const double ig = sigm(a[h] + r[h]), fg = sigm(a[H + h] + r[H + h]);
          const double gg = tanh(a[2 * H + h] + r[2 * H + h]), og = sigm(a[3 * H + h] + r[3 * H + h]);
          const double c = fg * tp->cprev[(size_t)s * BH + (size_t)b * H + h] + ig * gg;
          tp->cprev[(size_t)(s + 1) * BH + (size_t)b * H + h] = c;
          hv = og * tanh(c);
          gt[0] = ig; gt[BH] = fg; gt[2 * BH] = gg; gt[3 * BH] = og;
        } else {
          const double rg = sigm(a[h] + r[h]), zg = sigm(a[H + h] + r[H + h]);
          const double rn = r[2 * H + h];
          const double ng = tanh(a[2 * H + h] + rg * rn);
          tp->rn[(size_t)s * BH + (size_t)b * H + h] = rn;
          hv = (1.0 - zg) * ng + zg * hp[(size_t)b * H + h];
          gt[0] = rg; gt[BH] = zg; gt[2 * BH] = ng;
        }
        hn[(size_t)b * H + h] = hv;
        out[((size_t)t * B + b) * D * H + (size_t)dir * H + h] = hv;
      }
    }
  }
  free(a);
  free(r);
}

static rnn_tape rnn_tape_new(const flref_rnn* d) {
  const size_t BH = (size_t)d->B * d->hidden, T = d->T, G = rnn_gates(d->mode);
  rnn_tape tp;
  tp.hprev = (double*)calloc((T + 1) * BH, sizeof(double));
  tp.cprev = d->mode == 2 ? (double*)calloc((T + 1) * BH, sizeof(double)) : NULL;
  tp.gate = (double*)calloc(T * G * BH, sizeof(double));
  tp.rn = d->mode == 3 ? (double*)calloc(T * BH, sizeof(double)) : NULL;
  return tp;
}
static void rnn_tape_free(rnn_tape* tp) {
  free(tp->hprev); free(tp->cprev); free(tp->gate); free(tp->rn);
}

/* runs the whole stack; acts[l] = input of layer l (acts[layers] = y), tapes per pseudo-layer */
/* counter-based mask: two rounds of a 32-bit finaliser over (index, layer, seed); the top 24
 * bits as a uniform number in [0, 1) */
int flref_dropout_keep(uint32_t seed_lo, uint32_t seed_hi, uint32_t layer, uint32_t index, float dropout) {
  uint32_t h = index * 0x9E3779B1u ^ seed_lo;
  h ^= h >> 16; h *= 0x85EBCA6Bu; h ^= h >> 13; h *= 0xC2B2AE35u; h ^= h >> 16;
  h += seed_hi + layer * 0x632BE5ABu;
  h ^= h >> 16; h *= 0x85EBCA6Bu; h ^= h >> 13; h *= 0xC2B2AE35u; h ^= h >> 16;
  return (float)(h >> 8) * (1.0f / 16777216.0f) >= dropout;
}

static void rnn_stack_fwd(const flref_rnn* d, const float* x, const float* hx, const float* cx,
                          const float* w, double** acts, rnn_tape* tapes) {
  const int H = d->hidden, D = d->bidirectional ? 2 : 1, T = d->T, B = d->B;
  const size_t n0 = (size_t)T * B * d->input_size;
  acts[0] = (double*)malloc(sizeof(double) * n0);
  for (size_t i = 0; i < n0; ++i) acts[0][i] = x[i];
  for (int l = 0; l < d->layers; ++l) {
    const int64_t inl = l == 0 ? d->input_size : D * H;
    acts[l + 1] = (double*)calloc((size_t)T * B * D * H, sizeof(double));
    for (int dir = 0; dir < D; ++dir) {
      tapes[l * D + dir] = rnn_tape_new(d);
      rnn_layer_fwd(d, l * D + dir, acts[l], inl, w, hx, cx, acts[l + 1], &tapes[l * D + dir]);
    }
    /* dropout on what the next layer reads (the layer's own recurrence used the states in its tape) */
    if (d->dropout > 0.f && l + 1 < d->layers) {
      const size_t n = (size_t)T * B * D * H;
      const double scale = 1.0 / (1.0 - (double)d->dropout);
      for (size_t i = 0; i < n; ++i)
        acts[l + 1][i] = flref_dropout_keep(d->seed_lo, d->seed_hi, (uint32_t)l, (uint32_t)i, d->dropout) ? acts[l + 1][i] * scale : 0.0;
    }
  }
}

void flref_rnn_fwd(const flref_rnn* d, const float* x, const float* hx, const float* cx,
                   const float* w, float* y, float* hy, float* cy) {
  const int H = d->hidden, D = d->bidirectional ? 2 : 1, T = d->T, B = d->B, PL = d->layers * D;
  double** acts = (double**)calloc(d->layers + 1, sizeof(double*));
  rnn_tape* tapes = (rnn_tape*)calloc(PL, sizeof(rnn_tape));
  rnn_stack_fwd(d, x, hx, cx, w, acts, tapes);
  const size_t ny = (size_t)T * B * D * H, BH = (size_t)B * H;
  for (size_t i = 0; i < ny; ++i) y[i] = (float)acts[d->layers][i];
  for (int pl = 0; pl < PL; ++pl)
    for (size_t i = 0; i < BH; ++i) {
      hy[(size_t)pl * BH + i] = (float)tapes[pl].hprev[(size_t)T * BH + i];
      if (cy && d->mode == 2) cy[(size_t)pl * BH + i] = (float)tapes[pl].cprev[(size_t)T * BH + i];
    }
  for (int l = 0; l <= d->layers; ++l) free(acts[l]);
  for (int pl = 0; pl < PL; ++pl) rnn_tape_free(&tapes[pl]);
  free(acts);
  free(tapes);
}

void flref_rnn_bwd(const flref_rnn* d, const float* x, const float* hx, const float* cx,
                   const float* w, const float* dy, const float* dhy, const float* dcy,
                   float* dx, float* dhx, float* dcx, float* dw) {
  const int G = rnn_gates(d->mode), H = d->hidden, D = d->bidirectional ? 2 : 1, T = d->T, B = d->B;
  const int PL = d->layers * D;
  const size_t BH = (size_t)B * H;
  double** acts = (double**)calloc(d->layers + 1, sizeof(double*));
  rnn_tape* tapes = (rnn_tape*)calloc(PL, sizeof(rnn_tape));
  rnn_stack_fwd(d, x, hx, cx, w, acts, tapes);
  const int64_t nw = flref_rnn_param_count(d);
  double* gw = (double*)calloc((size_t)nw, sizeof(double));
  const size_t ny = (size_t)T * B * D * H;
  double* gout = (double*)calloc(ny, sizeof(double));          /* gradient of the layer output */
  if (dy) for (size_t i = 0; i < ny; ++i) gout[i] = dy[i];
  double* ga = (double*)malloc(sizeof(double) * G * H);        /* input-side pre-activation grads */
  double* gr = (double*)malloc(sizeof(double) * G * H);        /* recurrent-side */
  for (int l = d->layers - 1; l >= 0; --l) {
    const int64_t inl = l == 0 ? d->input_size : D * H;
    double* gin = (double*)calloc((size_t)T * B * inl, sizeof(double));
    for (int dir = 0; dir < D; ++dir) {
      const int pl = l * D + dir;
      const rnn_tape* tp = &tapes[pl];
      int64_t oW = 0, oR = 0, obW = 0, obR = 0;
      rnn_offsets(d, pl, &oW, &oR, &obW, &obR);
      double* gh = (double*)calloc(BH, sizeof(double));        /* dL/dh flowing back in time */
      double* gc = (double*)calloc(BH, sizeof(double));
      for (size_t i = 0; i < BH; ++i) {
        gh[i] = dhy ? dhy[(size_t)pl * BH + i] : 0.0;
        gc[i] = (dcy && d->mode == 2) ? dcy[(size_t)pl * BH + i] : 0.0;
      }
      double* ghp = (double*)malloc(sizeof(double) * BH);
      for (int s = T - 1; s >= 0; --s) {
        const int t = dir ? T - 1 - s : s;
        const double* hp = tp->hprev + (size_t)s * BH;
        for (size_t i = 0; i < BH; ++i) ghp[i] = 0.0;
        for (int b = 0; b < B; ++b) {
          const double* xin = acts[l] + ((size_t)t * B + b) * inl;
          for (int h = 0; h < H; ++h) {
            const size_t e = (size_t)b * H + h;
            const double* gt = tp->gate + (size_t)s * G * BH + e;
            const double go = gout[((size_t)t * B + b) * D * H + (size_t)dir * H + h] + gh[e];
            if (d->mode == 0 || d->mode == 1) {
              const double hv = gt[0];
              const double gp = d->mode == 0 ? (hv > 0 ? go : 0.0) : go * (1.0 - hv * hv);
              ga[h] = gr[h] = gp;
            } else if (d->mode == 2) {
              const double ig = gt[0], fg = gt[BH], gg = gt[2 * BH], og = gt[3 * BH];
              const double c = tp->cprev[(size_t)(s + 1) * BH + e], cp = tp->cprev[(size_t)s * BH + e];
              const double tc = tanh(c);
              const double dc = gc[e] + go * og * (1.0 - tc * tc);
              ga[h] = gr[h] = dc * gg * ig * (1.0 - ig);
              ga[H + h] = gr[H + h] = dc * cp * fg * (1.0 - fg);
              ga[2 * H + h] = gr[2 * H + h] = dc * ig * (1.0 - gg * gg);
              ga[3 * H + h] = gr[3 * H + h] = go * tc * og * (1.0 - og);
              gc[e] = dc * fg;
            } else {
              const double rg = gt[0], zg = gt[BH], ng = gt[2 * BH], rn = tp->rn[(size_t)s * BH + e];
              const double dn = go * (1.0 - zg) * (1.0 - ng * ng);
              ga[h] = gr[h] = dn * rn * rg * (1.0 - rg);
              ga[H + h] = gr[H + h] = go * (hp[e] - ng) * zg * (1.0 - zg);
              ga[2 * H + h] = dn;
              gr[2 * H + h] = dn * rg;
              ghp[e] += go * zg;
            }
          }
          for (int q = 0; q < G * H; ++q) {
            gw[obW + q] += ga[q];
            gw[obR + q] += gr[q];
            for (int64_t i = 0; i < inl; ++i) {
              gw[oW + (int64_t)q * inl + i] += ga[q] * xin[i];
              gin[((size_t)t * B + b) * inl + i] += ga[q] * (double)w[oW + (int64_t)q * inl + i];
            }
            for (int j = 0; j < H; ++j) {
              gw[oR + (int64_t)q * H + j] += gr[q] * hp[(size_t)b * H + j];
              ghp[(size_t)b * H + j] += gr[q] * (double)w[oR + (int64_t)q * H + j];
            }
          }
        }
        for (size_t i = 0; i < BH; ++i) gh[i] = ghp[i];
      }
      for (size_t i = 0; i < BH; ++i) {
        if (dhx) dhx[(size_t)pl * BH + i] = (float)gh[i];
        if (dcx && d->mode == 2) dcx[(size_t)pl * BH + i] = (float)gc[i];
      }
      free(gh); free(gc); free(ghp);
    }
    free(gout);
    gout = gin;
    /* gin is the gradient of what this layer read: the dropped output of the layer below */
    if (d->dropout > 0.f && l > 0) {
      const size_t n = (size_t)T * B * D * H;
      const double scale = 1.0 / (1.0 - (double)d->dropout);
      for (size_t i = 0; i < n; ++i)
        gout[i] = flref_dropout_keep(d->seed_lo, d->seed_hi, (uint32_t)(l - 1), (uint32_t)i, d->dropout) ? gout[i] * scale : 0.0;
    }
  }
  const size_t nx = (size_t)T * B * d->input_size;
  for (size_t i = 0; i < nx; ++i) dx[i] = (float)gout[i];
  for (int64_t i = 0; i < nw; ++i) dw[i] = (float)gw[i];
  free(gout); free(ga); free(gr); free(gw);
  for (int l = 0; l <= d->layers; ++l) free(acts[l]);
  for (int pl = 0; pl < PL; ++pl) rnn_tape_free(&tapes[pl]);
  free(acts);
  free(tapes);
}
