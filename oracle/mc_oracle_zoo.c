/*
 * mc_oracle_zoo.c — CPU restatement of the less common Mini-Caffe layers.
 *
 * TEST INFRASTRUCTURE ONLY, like mc_oracle.c: the checker for the HIP path.
 * Nothing in the product library links, loads or calls it.
 *
 * Each function follows the reference's CPU code in its order of operations and
 * cites it (paths relative to the reference checkout).  The reference routes
 * vsPowx / vsExp / vsLn / vsSqr / vsAbs through src/util/mkl_alternate.hpp:22-58,
 * plain loops over the <math.h> functions on floats.
 *
 * How each function is pinned (tests/test_oracle_zoo.py):
 *   bn                    float64 closed form with non-trivial multiplier blob
 *                         (tells it from BatchNorm: no root, no eps)
 *   conv_dw               torch conv2d(groups = channels) in float64 and the
 *                         grouped im2col+gemm oracle
 *   power / exp / log     numpy float64 closed forms incl. the constant-output
 *                         special cases and base != e
 *   absval / bnll / elu / threshold / prelu   numpy closed forms
 *   lrn (both regions)    float64 brute force over the clipped window; the padded
 *                         divisor of the within-channel average
 *   argmax                numpy argsort on distinct values, hand-made ties, all
 *                         three output layouts
 *   reduction / mvn       numpy float64 (eps outside the root for mvn)
 *   embed                 numpy fancy indexing
 *   shuffle_channel       numpy reshape/transposition; shuffle(g) then
 *                         shuffle(C/g) is the identity
 * Sums that the reference hands to BLAS (sdot, sasum, sgemv) are accumulated here
 * in index order: parity there is the stated tolerance, not bit equality.
 */
#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* BNLayer::Forward_cpu (src/layers/bn_layer.cpp:77-147): subtract the stored mean,
 * multiply by blobs[3] as it is, multiply by the slope, add the bias — four passes,
 * four roundings.  The broadcast gemms have inner dimension 1 and are exact. */
void orc_bn(int num, int channels, int spatial, const float* x, const float* slope,
            const float* bias, const float* mean, const float* mult, float* y) {
  for (int n = 0; n < num; ++n)
    for (int c = 0; c < channels; ++c) {
      const float* xp = x + ((size_t)n * channels + c) * spatial;
      float* yp = y + ((size_t)n * channels + c) * spatial;
      const float neg_mean = -1.f * mean[c];
      for (int i = 0; i < spatial; ++i) {
        float t = xp[i] + neg_mean;
        t = t * mult[c];
        t = t * slope[c];
        yp[i] = t + bias[c];
      }
    }
}

/* ConvolutionDepthwiseLayer::Forward_cpu (src/layers/conv_dw_layer.cpp:105-158):
 * direct sum over the taps in (kh, kw) order starting from 0, bias added after. */
void orc_conv_dw(int num, int channels, int H, int W, int kh, int kw, int sh, int sw, int ph,
                 int pw, int dh, int dw, const float* x, const float* w, const float* bias,
                 float* y) {
  const int Ho = (H + 2 * ph - (dh * (kh - 1) + 1)) / sh + 1;
  const int Wo = (W + 2 * pw - (dw * (kw - 1) + 1)) / sw + 1;
  for (int n = 0; n < num; ++n)
    for (int c = 0; c < channels; ++c)
      for (int h = 0; h < Ho; ++h)
        for (int q = 0; q < Wo; ++q) {
          const float* wt = w + (size_t)c * kh * kw;
          float value = 0;
          for (int i = 0; i < kh; ++i)
            for (int j = 0; j < kw; ++j) {
              const int h_in = -ph + h * sh + i * dh;
              const int w_in = -pw + q * sw + j * dw;
              if (h_in >= 0 && h_in < H && w_in >= 0 && w_in < W)
                value += (*wt) * x[(((size_t)n * channels + c) * H + h_in) * W + w_in];
              ++wt;
            }
          float* out = y + (((size_t)n * channels + c) * Ho + h) * Wo + q;
          *out = value;
          if (bias) *out += bias[c];
        }
}

/* PowerLayer::Forward_cpu (src/layers/power_layer.cpp:17-40). */
void orc_power(size_t n, const float* x, float scale, float shift, float power, float* y) {
  const float diff_scale = power * scale;
  if (diff_scale == 0.f) {
    const float value = (power == 0) ? 1 : powf(shift, power);
    for (size_t i = 0; i < n; ++i) y[i] = value;
    return;
  }
  for (size_t i = 0; i < n; ++i) y[i] = x[i];
  if (scale != 1.f)
    for (size_t i = 0; i < n; ++i) y[i] *= scale;
  if (shift != 0.f)
    for (size_t i = 0; i < n; ++i) y[i] += shift;
  if (power != 1.f)
    for (size_t i = 0; i < n; ++i) y[i] = powf(y[i], power);
}

/* ExpLayer (src/layers/exp_layer.cpp:8-45). */
void orc_exp_layer(size_t n, const float* x, float base, float scale, float shift, float* y) {
  const float log_base = (base == -1.f) ? 1 : logf(base);
  const float inner_scale = log_base * scale;
  const float outer_scale =
      (shift == 0.f) ? 1 : ((base != -1.f) ? powf(base, shift) : expf(shift));
  if (inner_scale == 1.f) {
    for (size_t i = 0; i < n; ++i) y[i] = expf(x[i]);
  } else {
    for (size_t i = 0; i < n; ++i) y[i] = x[i] * inner_scale;
    for (size_t i = 0; i < n; ++i) y[i] = expf(y[i]);
  }
  if (outer_scale != 1.f)
    for (size_t i = 0; i < n; ++i) y[i] *= outer_scale;
}

/* LogLayer (src/layers/log_layer.cpp:8-54). */
void orc_log_layer(size_t n, const float* x, float base, float scale, float shift, float* y) {
  const float log_base = (base == -1.f) ? 1 : logf(base);
  const float base_scale = 1.f / log_base;
  if (scale == 1.f && shift == 0.f) {
    for (size_t i = 0; i < n; ++i) y[i] = logf(x[i]);
  } else {
    for (size_t i = 0; i < n; ++i) y[i] = x[i];
    if (scale != 1.f)
      for (size_t i = 0; i < n; ++i) y[i] *= scale;
    if (shift != 0.f)
      for (size_t i = 0; i < n; ++i) y[i] += shift;
    for (size_t i = 0; i < n; ++i) y[i] = logf(y[i]);
  }
  if (base_scale != 1.f)
    for (size_t i = 0; i < n; ++i) y[i] *= base_scale;
}

/* AbsValLayer::Forward_cpu (src/layers/absval_layer.cpp:8-13). */
void orc_absval(size_t n, const float* x, float* y) {
  for (size_t i = 0; i < n; ++i) y[i] = fabsf(x[i]);
}

/* BNLLLayer::Forward_cpu (src/layers/bnll_layer.cpp:8-18): the literal 1. makes the
 * inner arithmetic double. */
void orc_bnll(size_t n, const float* x, float* y) {
  for (size_t i = 0; i < n; ++i)
    y[i] = x[i] > 0 ? (float)(x[i] + log(1. + exp(-(double)x[i])))
                    : (float)log(1. + exp((double)x[i]));
}

/* ELULayer::Forward_cpu (src/layers/elu_layer.cpp:8-18). */
void orc_elu(size_t n, const float* x, float alpha, float* y) {
  for (size_t i = 0; i < n; ++i) {
    const float pos = x[i] > 0.f ? x[i] : 0.f;
    const float neg = x[i] < 0.f ? x[i] : 0.f;
    y[i] = pos + alpha * (expf(neg) - 1);
  }
}

/* ThresholdLayer::Forward_cpu (src/layers/threshold_layer.cpp:13-21). */
void orc_threshold(size_t n, const float* x, float threshold, float* y) {
  for (size_t i = 0; i < n; ++i) y[i] = (x[i] > threshold) ? 1 : 0;
}

/* PReLULayer::Forward_cpu (src/layers/prelu_layer.cpp:50-84). */
void orc_prelu(int num, int channels, int dim, const float* x, const float* slope, int shared,
               float* y) {
  for (int n = 0; n < num; ++n)
    for (int c = 0; c < channels; ++c) {
      const float s = slope[shared ? 0 : c];
      for (int k = 0; k < dim; ++k) {
        const float v = *x++;
        *y++ = (v > 0.f ? v : 0.f) + s * (v < 0.f ? v : 0.f);
      }
    }
}

/* LRNLayer::CrossChannelForward_cpu (src/layers/lrn_layer.cpp:112-155): the scale of
 * channel 0 is k plus the first window, later channels copy the previous scale,
 * add the entering and subtract the leaving squared value (alpha/size folded into
 * each axpy); output = scale^-beta * x. */
void orc_lrn_across(int num, int channels, int H, int W, int size, float alpha, float beta,
                    float k, const float* x, float* y) {
  const int spatial = H * W;
  const int pre_pad = (size - 1) / 2;
  const float alpha_over_size = alpha / size;
  float* padded = (float*)calloc((size_t)(channels + size - 1) * spatial, sizeof(float));
  float* scale = (float*)malloc((size_t)channels * spatial * sizeof(float));
  for (int n = 0; n < num; ++n) {
    const float* xn = x + (size_t)n * channels * spatial;
    float* yn = y + (size_t)n * channels * spatial;
    for (size_t i = 0; i < (size_t)channels * spatial; ++i)
      padded[(size_t)pre_pad * spatial + i] = xn[i] * xn[i];
    for (int i = 0; i < channels * spatial; ++i) scale[i] = k;
    for (int c = 0; c < size; ++c)
      for (int i = 0; i < spatial; ++i) scale[i] += alpha_over_size * padded[(size_t)c * spatial + i];
    for (int c = 1; c < channels; ++c) {
      float* sc = scale + (size_t)c * spatial;
      memcpy(sc, sc - spatial, spatial * sizeof(float));
      for (int i = 0; i < spatial; ++i)
        sc[i] += alpha_over_size * padded[(size_t)(c + size - 1) * spatial + i];
      for (int i = 0; i < spatial; ++i)
        sc[i] += -alpha_over_size * padded[(size_t)(c - 1) * spatial + i];
    }
    for (size_t i = 0; i < (size_t)channels * spatial; ++i) yn[i] = powf(scale[i], -beta);
    for (size_t i = 0; i < (size_t)channels * spatial; ++i) yn[i] = yn[i] * xn[i];
  }
  free(padded);
  free(scale);
}

/* ArgMaxLayer::Forward_cpu (src/layers/argmax_layer.cpp:56-93): per line, the top_k
 * first of (value, index) pairs sorted by std::greater on the pair.
 * layout 0: indices, 1: values (both [.., top_k, axis_dist]); 2: indices then values
 * per instance (no axis, out_max_val). */
typedef struct {
  float v;
  int i;
} orc_pair;
static int pair_greater(const void* a, const void* b) {
  const orc_pair* p = (const orc_pair*)a;
  const orc_pair* q = (const orc_pair*)b;
  if (p->v > q->v) return -1;
  if (p->v < q->v) return 1;
  return (p->i > q->i) ? -1 : (p->i < q->i);
}
void orc_argmax(int count, int dim, int axis_dist, int top_k, int layout, const float* x,
                float* y) {
  const int num = count / dim;
  orc_pair* v = (orc_pair*)malloc((size_t)dim * sizeof(orc_pair));
  for (int i = 0; i < num; ++i) {
    for (int j = 0; j < dim; ++j) {
      v[j].v = x[((size_t)(i / axis_dist) * dim + j) * axis_dist + i % axis_dist];
      v[j].i = j;
    }
    qsort(v, dim, sizeof(orc_pair), pair_greater);
    for (int j = 0; j < top_k; ++j) {
      if (layout == 2) {
        y[2 * (size_t)i * top_k + j] = (float)v[j].i;
        y[2 * (size_t)i * top_k + top_k + j] = v[j].v;
      } else {
        y[((size_t)(i / axis_dist) * top_k + j) * axis_dist + i % axis_dist] =
            layout == 1 ? v[j].v : (float)v[j].i;
      }
    }
  }
  free(v);
}

/* ReductionLayer::Forward_cpu (src/layers/reduction_layer.cpp:38-72); op values as
 * in ReductionParameter: 1 SUM, 2 ASUM, 3 SUMSQ, 4 MEAN. */
void orc_reduction(int op, int num, int dim, float coeff, const float* x, float* y) {
  if (op == 4) coeff /= dim;
  for (int i = 0; i < num; ++i) {
    const float* xr = x + (size_t)i * dim;
    float acc = 0.f;
    for (int d = 0; d < dim; ++d)
      acc += op == 2 ? fabsf(xr[d]) : (op == 3 ? xr[d] * xr[d] : 1.f * xr[d]);
    y[i] = acc;
  }
  if (coeff != 1.f)
    for (int i = 0; i < num; ++i) y[i] *= coeff;
}

/* MVNLayer::Forward_cpu (src/layers/mvn_layer.cpp:36-75): mean by gemv with
 * alpha = 1/dim, x - mean, then (optionally) divided by
 * powf(mean((x-mean)^2), 0.5) + eps. */
void orc_mvn(int num, int dim, int normalize_variance, float eps, const float* x, float* y) {
  const float alpha = (float)(1. / dim);
  for (int r = 0; r < num; ++r) {
    const float* xr = x + (size_t)r * dim;
    float* yr = y + (size_t)r * dim;
    float s = 0.f;
    for (int d = 0; d < dim; ++d) s += xr[d];
    const float neg_mean = -1.f * (alpha * s);
    for (int d = 0; d < dim; ++d) yr[d] = xr[d] + neg_mean;
    if (normalize_variance) {
      float q = 0.f;
      for (int d = 0; d < dim; ++d) q += powf(yr[d], 2.f);
      float var = alpha * q;
      var = powf(var, 0.5f);
      var += eps;
      for (int d = 0; d < dim; ++d) yr[d] = yr[d] / var;
    }
  }
}

/* EmbedLayer::Forward_cpu (src/layers/embed_layer.cpp:62-79). */
void orc_embed(int M, int N, const float* x, const float* weight, const float* bias, float* y) {
  for (int n = 0; n < M; ++n) {
    const int index = (int)x[n];
    memcpy(y + (size_t)n * N, weight + (size_t)index * N, N * sizeof(float));
  }
  if (bias)
    for (int n = 0; n < M; ++n)
      for (int j = 0; j < N; ++j) y[(size_t)n * N + j] += 1.f * bias[j];
}

/* ShuffleChannelLayer::Forward_cpu (src/layers/shuffle_channel_layer.cpp:17-58):
 * channel i*columns + j moves to j*rows + i, rows = group. */
void orc_shuffle_channel(int num, int channels, int spatial, int group, const float* x,
                         float* y) {
  const int rows = group, columns = channels / group;
  for (int n = 0; n < num; ++n)
    for (int i = 0; i < rows; ++i)
      for (int j = 0; j < columns; ++j)
        memcpy(y + ((size_t)n * channels + j * rows + i) * spatial,
               x + ((size_t)n * channels + i * columns + j) * spatial, spatial * sizeof(float));
}
