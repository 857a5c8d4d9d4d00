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
