/*
 * mc_oracle.c — CPU restatement of Mini-Caffe's forward arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, what the
 * reference's CPU layers compute, in the reference's order of operations.  It
 * is the checker for the HIP path: only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load it.  Nothing in the product library
 * links, loads or calls it.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference checkout).
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   im2col / col2im / gemm            bit-exact against oracle/_ref (the
 *                                     reference's own im2col.cpp and
 *                                     math_functions.cpp compiled as they lie)
 *   conv / deconv / inner product     float64 brute-force direct sums, torch
 *                                     conv2d / conv_transpose2d, the adjoint
 *                                     identity <conv(x),y> = <x,deconv(y)>
 *   exp / powx / div / scale helpers  bit-exact against oracle/_ref
 *   batch norm / scale / bias / relu  closed forms in float64
 *   pooling                           independent brute force incl. ceil mode
 *                                     and the padded-average divisor
 *   eltwise / softmax                 numpy closed forms
 * The BLAS boundary itself (summation order inside OpenBLAS sgemm/sgemv) has
 * no golden vector in the reference: parity there is the stated tolerance, not
 * bit equality.
 */
#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---- GEMM ---------------------------------------------------------------- */

/* cblas_sgemm signature (row-major = 101, NoTrans = 111, Trans = 112). */
typedef void (*cblas_sgemm_fn)(int order, int transa, int transb, int M, int N, int K,
                               float alpha, const float* A, int lda, const float* B, int ldb,
                               float beta, float* C, int ldc);
static cblas_sgemm_fn g_sgemm = 0;

/* Lets the harness plug a real CBLAS (the reference links OpenBLAS:
 * src/util/math_functions.cpp:8-16). 0 restores the built-in loops. */
void orc_set_sgemm(void* fn) { g_sgemm = (cblas_sgemm_fn)fn; }
int orc_has_blas(void) { return g_sgemm != 0; }

/* caffe_cpu_gemm (src/util/math_functions.cpp:8-16): row-major
 * C = alpha*op(A)*op(B) + beta*C, lda = K or M, ldb = N or K, ldc = N. */
void orc_gemm(int transa, int transb, int M, int N, int K, float alpha, const float* A,
              const float* B, float beta, float* C) {
  const int lda = transa ? M : K;
  const int ldb = transb ? K : N;
  if (g_sgemm) {
    g_sgemm(101, transa ? 112 : 111, transb ? 112 : 111, M, N, K, alpha, A, lda, B, ldb, beta, C,
            N);
    return;
  }
  for (int i = 0; i < M; ++i) {
    float* c = C + (size_t)i * N;
    if (beta == 0.f) {
      memset(c, 0, sizeof(float) * N);
    } else if (beta != 1.f) {
      for (int j = 0; j < N; ++j) c[j] *= beta;
    }
    for (int k = 0; k < K; ++k) {
      const float a = alpha * (transa ? A[(size_t)k * lda + i] : A[(size_t)i * lda + k]);
      if (!transb) {
        const float* b = B + (size_t)k * ldb;
        for (int j = 0; j < N; ++j) c[j] += a * b[j];
      } else {
        for (int j = 0; j < N; ++j) c[j] += a * B[(size_t)j * ldb + k];
      }
    }
  }
}

/* ---- im2col / col2im ------------------------------------------------------ */

static int out_extent(int in, int pad, int dil, int k, int stride) {
  return (in + 2 * pad - (dil * (k - 1) + 1)) / stride + 1;
}

/* im2col_cpu (src/util/im2col.cpp:19-55): col[(c*kh+i)*kw+j][ho][wo] =
 * im[c][ho*s-p+i*d][wo*s-p+j*d], zero outside the image. */
void orc_im2col(const float* im, int C, int H, int W, int kh, int kw, int ph, int pw, int sh,
                int sw, int dh, int dw, float* col) {
  const int Ho = out_extent(H, ph, dh, kh, sh), Wo = out_extent(W, pw, dw, kw, sw);
  for (int c = 0; c < C; ++c)
    for (int i = 0; i < kh; ++i)
      for (int j = 0; j < kw; ++j) {
        float* dst = col + ((size_t)(c * kh + i) * kw + j) * Ho * Wo;
        for (int ho = 0; ho < Ho; ++ho) {
          const int h = ho * sh - ph + i * dh;
          for (int wo = 0; wo < Wo; ++wo) {
            const int w = wo * sw - pw + j * dw;
            const int inside = (unsigned)h < (unsigned)H && (unsigned)w < (unsigned)W;
            dst[ho * Wo + wo] = inside ? im[((size_t)c * H + h) * W + w] : 0.f;
          }
        }
      }
}

/* col2im_cpu (src/util/im2col.cpp:153-187): zero the image, then add every
 * column entry to the pixel it was unfolded from, in (c, i, j, ho, wo) order. */
void orc_col2im(const float* col, int C, int H, int W, int kh, int kw, int ph, int pw, int sh,
                int sw, int dh, int dw, float* im) {
  const int Ho = out_extent(H, ph, dh, kh, sh), Wo = out_extent(W, pw, dw, kw, sw);
  memset(im, 0, sizeof(float) * (size_t)C * H * W);
  for (int c = 0; c < C; ++c)
    for (int i = 0; i < kh; ++i)
      for (int j = 0; j < kw; ++j) {
        const float* src = col + ((size_t)(c * kh + i) * kw + j) * Ho * Wo;
        for (int ho = 0; ho < Ho; ++ho) {
          const int h = ho * sh - ph + i * dh;
          if ((unsigned)h >= (unsigned)H) continue;
          for (int wo = 0; wo < Wo; ++wo) {
            const int w = wo * sw - pw + j * dw;
            if ((unsigned)w < (unsigned)W) im[((size_t)c * H + h) * W + w] += src[ho * Wo + wo];
          }
        }
      }
}

/* ---- Convolution / Deconvolution / InnerProduct ---------------------------- */

typedef struct {
  int channels_in, height_in, width_in, channels_out;
  int kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w;
  int group;
  int transposed;
} orc_conv_geom;

void orc_conv_output_shape(const orc_conv_geom* g, int* Ho, int* Wo) {
  const int eh = g->dilation_h * (g->kernel_h - 1) + 1, ew = g->dilation_w * (g->kernel_w - 1) + 1;
  if (!g->transposed) { /* src/layers/conv_layer.cpp:12-25 */
    *Ho = (g->height_in + 2 * g->pad_h - eh) / g->stride_h + 1;
    *Wo = (g->width_in + 2 * g->pad_w - ew) / g->stride_w + 1;
  } else { /* src/layers/deconv_layer.cpp:11-25 */
    *Ho = g->stride_h * (g->height_in - 1) + eh - 2 * g->pad_h;
    *Wo = g->stride_w * (g->width_in - 1) + ew - 2 * g->pad_w;
  }
}

/* forward_cpu_bias (src/layers/base_conv_layer.cpp:273-278):
 * top (Cout x HoWo) += bias (Cout x 1) * ones (1 x HoWo), a rank-1 gemm. */
static void conv_bias(float* top, const float* bias, const float* ones, int Cout, int spatial) {
  orc_gemm(0, 0, Cout, spatial, 1, 1.f, bias, ones, 1.f, top);
}

/* ConvolutionLayer::Forward_cpu (src/layers/conv_layer.cpp:27-42) with
 * forward_cpu_gemm (base_conv_layer.cpp:254-271): per image, im2col unless the
 * filter is 1x1/s1/p0 (:110-115), then one gemm per group with beta = 0.
 * weights [Cout, Cin/g, kh, kw]; bias may be NULL. */
void orc_conv_forward(const orc_conv_geom* g, int num, const float* bottom, const float* weights,
                      const float* bias, float* top) {
  int Ho, Wo;
  orc_conv_output_shape(g, &Ho, &Wo);
  const int spatial = Ho * Wo;
  const int kdim = (g->channels_in / g->group) * g->kernel_h * g->kernel_w;
  const int Mg = g->channels_out / g->group;
  const size_t bottom_dim = (size_t)g->channels_in * g->height_in * g->width_in;
  const size_t top_dim = (size_t)g->channels_out * spatial;
  const int is_1x1 = g->kernel_h == 1 && g->kernel_w == 1 && g->stride_h == 1 &&
                     g->stride_w == 1 && g->pad_h == 0 && g->pad_w == 0;
  float* ones = (float*)malloc(sizeof(float) * spatial);
  for (int i = 0; i < spatial; ++i) ones[i] = 1.f;
#pragma omp parallel if (!g_sgemm)
  {
    float* col = is_1x1 ? 0 : (float*)malloc(sizeof(float) * (size_t)kdim * g->group * spatial);
#pragma omp for schedule(dynamic)
    for (int n = 0; n < num; ++n) {
      const float* x = bottom + n * bottom_dim;
      float* y = top + n * top_dim;
      const float* colp = x;
      if (!is_1x1) {
        orc_im2col(x, g->channels_in, g->height_in, g->width_in, g->kernel_h, g->kernel_w,
                   g->pad_h, g->pad_w, g->stride_h, g->stride_w, g->dilation_h, g->dilation_w,
                   col);
        colp = col;
      }
      for (int gi = 0; gi < g->group; ++gi)
        orc_gemm(0, 0, Mg, spatial, kdim, 1.f, weights + (size_t)gi * Mg * kdim,
                 colp + (size_t)gi * kdim * spatial, 0.f, y + (size_t)gi * Mg * spatial);
      if (bias) conv_bias(y, bias, ones, g->channels_out, spatial);
    }
    free(col);
  }
  free(ones);
}

/* DeconvolutionLayer::Forward_cpu (src/layers/deconv_layer.cpp:27-42) with
 * backward_cpu_gemm (base_conv_layer.cpp:280-296): per image and group,
 * col = W_g^T * x_g (gemm with A transposed), then col2im into the top, then
 * the bias.  weights [Cin, Cout/g, kh, kw].  In the reference's bookkeeping the
 * roles of "in" and "out" swap (reverse_dimensions), so the gemm has
 * M = (Cout/g)*kh*kw, N = Hin*Win, K = Cin/g. */
void orc_deconv_forward(const orc_conv_geom* g, int num, const float* bottom,
                        const float* weights, const float* bias, float* top) {
  int Ho, Wo;
  orc_conv_output_shape(g, &Ho, &Wo);
  const int in_spatial = g->height_in * g->width_in;
  const int Cg_out = g->channels_out / g->group;
  const int Cg_in = g->channels_in / g->group;
  const int kdim = Cg_out * g->kernel_h * g->kernel_w; /* rows of col per group */
  const size_t bottom_dim = (size_t)g->channels_in * in_spatial;
  const size_t top_dim = (size_t)g->channels_out * Ho * Wo;
  const int is_1x1 = g->kernel_h == 1 && g->kernel_w == 1 && g->stride_h == 1 &&
                     g->stride_w == 1 && g->pad_h == 0 && g->pad_w == 0;
  const int spatial = Ho * Wo;
  float* ones = (float*)malloc(sizeof(float) * spatial);
  for (int i = 0; i < spatial; ++i) ones[i] = 1.f;
#pragma omp parallel if (!g_sgemm)
  {
    float* col = is_1x1 ? 0 : (float*)malloc(sizeof(float) * (size_t)kdim * g->group * in_spatial);
#pragma omp for schedule(dynamic)
    for (int n = 0; n < num; ++n) {
      const float* x = bottom + n * bottom_dim;
      float* y = top + n * top_dim;
      float* colp = is_1x1 ? y : col;
      for (int gi = 0; gi < g->group; ++gi)
        orc_gemm(1, 0, kdim, in_spatial, Cg_in, 1.f, weights + (size_t)gi * Cg_in * kdim,
                 x + (size_t)gi * Cg_in * in_spatial, 0.f, colp + (size_t)gi * kdim * in_spatial);
      if (!is_1x1)
        orc_col2im(col, g->channels_out, Ho, Wo, g->kernel_h, g->kernel_w, g->pad_h, g->pad_w,
                   g->stride_h, g->stride_w, g->dilation_h, g->dilation_w, y);
      if (bias) conv_bias(y, bias, ones, g->channels_out, spatial);
    }
    free(col);
  }
  free(ones);
}

/* InnerProductLayer::Forward_cpu (src/layers/inner_product_layer.cpp:80-93):
 * top (M x N) = bottom (M x K) * W^T, W is N x K (K x N when transpose), then
 * top += ones (M x 1) * bias (1 x N). */
void orc_inner_product(int M, int N, int K, const float* bottom, const float* weights,
                       const float* bias, int transpose, float* top) {
  orc_gemm(0, transpose ? 0 : 1, M, N, K, 1.f, bottom, weights, 0.f, top);
  if (bias) {
    float* ones = (float*)malloc(sizeof(float) * M);
    for (int i = 0; i < M; ++i) ones[i] = 1.f;
    orc_gemm(0, 0, M, N, 1, 1.f, ones, bias, 1.f, top);
    free(ones);
  }
}

/* ---- small math helpers (src/util/mkl_alternate.hpp:22-58) ---------------- */

/* That header includes <math.h>, so exp/pow on float arguments resolve to the
 * float overloads. */
void orc_exp(int n, const float* a, float* y) {
  for (int i = 0; i < n; ++i) y[i] = expf(a[i]);
}
void orc_powx(int n, const float* a, float b, float* y) {
  for (int i = 0; i < n; ++i) y[i] = powf(a[i], b);
}

/* ---- BatchNorm (src/layers/batch_norm_layer.cpp:73-136) ------------------- */

/* blob0 = mean sum, blob1 = variance sum, blob2[0] = moving-average factor.
 * use_global_stats: mean = blob0/blob2, var = blob1/blob2 (both 0 when blob2 is 0).
 * Otherwise mean and E[(x-mean)^2] over num*spatial per channel, as two
 * reductions each (over the spatial extent with alpha = 1/(num*spatial), then
 * over the batch).  Output (x - mean) / powf(var + eps, 0.5f). */
void orc_batch_norm(int num, int channels, int spatial, const float* bottom, const float* blob0,
                    const float* blob1, const float* blob2, int use_global_stats, float eps,
                    float* top) {
  float* mean = (float*)calloc(channels, sizeof(float));
  float* var = (float*)calloc(channels, sizeof(float));
  const size_t count = (size_t)num * channels * spatial;
  if (top != bottom) memcpy(top, bottom, sizeof(float) * count);
  if (use_global_stats) {
    const float factor = blob2[0] == 0.f ? 0.f : 1.f / blob2[0];
    for (int c = 0; c < channels; ++c) {
      mean[c] = factor * blob0[c];
      var[c] = factor * blob1[c];
    }
  } else {
    const float alpha = (float)(1. / ((double)num * spatial));
    for (int n = 0; n < num; ++n)
      for (int c = 0; c < channels; ++c) {
        const float* x = bottom + ((size_t)n * channels + c) * spatial;
        float s = 0.f;
        for (int i = 0; i < spatial; ++i) s += x[i];
        mean[c] += alpha * s;
      }
  }
  for (int n = 0; n < num; ++n)
    for (int c = 0; c < channels; ++c) {
      float* y = top + ((size_t)n * channels + c) * spatial;
      for (int i = 0; i < spatial; ++i) y[i] = y[i] + (-1.f * mean[c]);
    }
  if (!use_global_stats) {
    const float alpha = (float)(1. / ((double)num * spatial));
    for (int n = 0; n < num; ++n)
      for (int c = 0; c < channels; ++c) {
        const float* y = top + ((size_t)n * channels + c) * spatial;
        float s = 0.f;
        for (int i = 0; i < spatial; ++i) s += powf(y[i], 2.f);
        var[c] += alpha * s;
      }
  }
  for (int c = 0; c < channels; ++c) var[c] = powf(var[c] + eps, 0.5f);
  for (int n = 0; n < num; ++n)
    for (int c = 0; c < channels; ++c) {
      float* y = top + ((size_t)n * channels + c) * spatial;
      for (int i = 0; i < spatial; ++i) y[i] = y[i] / var[c];
    }
  free(mean);
  free(var);
}

/* ---- Scale / Bias (src/layers/scale_layer.cpp:96-114, bias_layer.cpp:68-83) */

/* top[n][d][i] = bottom[n][d][i] * scale[d], then += bias[d] when bias != NULL. */
void orc_scale(int outer, int scale_dim, int inner, const float* bottom, const float* scale,
               const float* bias, float* top) {
  for (int n = 0; n < outer; ++n)
    for (int d = 0; d < scale_dim; ++d) {
      const size_t o = ((size_t)n * scale_dim + d) * inner;
      for (int i = 0; i < inner; ++i) top[o + i] = scale[d] * bottom[o + i];
    }
  if (bias)
    for (int n = 0; n < outer; ++n)
      for (int d = 0; d < scale_dim; ++d) {
        const size_t o = ((size_t)n * scale_dim + d) * inner;
        for (int i = 0; i < inner; ++i) top[o + i] += bias[d];
      }
}

void orc_bias(int outer, int bias_dim, int inner, const float* bottom, const float* bias,
              float* top) {
  const size_t count = (size_t)outer * bias_dim * inner;
  if (top != bottom) memcpy(top, bottom, sizeof(float) * count);
  for (int n = 0; n < outer; ++n)
    for (int d = 0; d < bias_dim; ++d) {
      const size_t o = ((size_t)n * bias_dim + d) * inner;
      for (int i = 0; i < inner; ++i) top[o + i] += bias[d];
    }
}

/* ---- activations ---------------------------------------------------------- */

/* ReLULayer::Forward_cpu (src/layers/relu_layer.cpp:12-30): a slope with
 * |slope| < 1e-6 counts as zero. */
void orc_relu(size_t n, const float* x, float slope, float* y) {
  if (fabsf(slope) < 1e-6) {
    for (size_t i = 0; i < n; ++i) y[i] = x[i] > 0.f ? x[i] : 0.f;
  } else {
    for (size_t i = 0; i < n; ++i)
      y[i] = (x[i] > 0.f ? x[i] : 0.f) + slope * (x[i] < 0.f ? x[i] : 0.f);
  }
}

/* TanHLayer::Forward_cpu (src/layers/tanh_layer.cpp:14-22): the file includes
 * only <vector>, so the unqualified tanh(float) is ::tanh(double), narrowed. */
void orc_tanh(size_t n, const float* x, float* y) {
  for (size_t i = 0; i < n; ++i) y[i] = (float)tanh((double)x[i]);
}

/* sigmoid (src/layers/sigmoid_layer.cpp:12-14): 1. / (1. + exp(-x)).  Only
 * <cmath> is included, which leaves ::exp(double) as the one candidate for the
 * unqualified call, so the whole expression is evaluated in double and narrowed.
 * (Whether a generated protobuf header drags <math.h> in and so selects the
 * float overloads for tanh/exp cannot be checked without that header; the two
 * readings differ by at most one float ulp.) */
void orc_sigmoid(size_t n, const float* x, float* y) {
  for (size_t i = 0; i < n; ++i) y[i] = (float)(1. / (1. + exp((double)(-x[i]))));
}

/* ---- Pooling (src/layers/pooling_layer.cpp:81-189) ------------------------ */

void orc_pooling_output_shape(int H, int W, int kh, int kw, int sh, int sw, int ph, int pw,
                              int* Ho, int* Wo) {
  int ho = (int)ceil((float)(H + 2 * ph - kh) / sh) + 1;
  int wo = (int)ceil((float)(W + 2 * pw - kw) / sw) + 1;
  if (ph || pw) {
    if ((ho - 1) * sh >= H + ph) --ho;
    if ((wo - 1) * sw >= W + pw) --wo;
  }
  *Ho = ho;
  *Wo = wo;
}

/* method 0 = MAX (start from -FLT_MAX, window clipped to the image),
 * 1 = AVE (sum over the clipped window, divided by the window area clipped to
 * the padded extent). */
void orc_pooling(int method, int planes, int H, int W, int kh, int kw, int sh, int sw, int ph,
                 int pw, const float* bottom, float* top) {
  int Ho, Wo;
  orc_pooling_output_shape(H, W, kh, kw, sh, sw, ph, pw, &Ho, &Wo);
#pragma omp parallel for
  for (int pl = 0; pl < planes; ++pl) {
    const float* x = bottom + (size_t)pl * H * W;
    float* y = top + (size_t)pl * Ho * Wo;
    for (int oh = 0; oh < Ho; ++oh)
      for (int ow = 0; ow < Wo; ++ow) {
        int hs = oh * sh - ph, ws = ow * sw - pw;
        if (method == 0) {
          int he = hs + kh < H ? hs + kh : H, we = ws + kw < W ? ws + kw : W;
          if (hs < 0) hs = 0;
          if (ws < 0) ws = 0;
          float m = -FLT_MAX;
          for (int h = hs; h < he; ++h)
            for (int w = ws; w < we; ++w)
              if (x[h * W + w] > m) m = x[h * W + w];
          y[oh * Wo + ow] = m;
        } else {
          int he = hs + kh < H + ph ? hs + kh : H + ph;
          int we = ws + kw < W + pw ? ws + kw : W + pw;
          const int area = (he - hs) * (we - ws);
          if (hs < 0) hs = 0;
          if (ws < 0) ws = 0;
          if (he > H) he = H;
          if (we > W) we = W;
          float s = 0.f;
          for (int h = hs; h < he; ++h)
            for (int w = ws; w < we; ++w) s += x[h * W + w];
          y[oh * Wo + ow] = s / area;
        }
      }
  }
}

/* ---- Eltwise (src/layers/eltwise_layer.cpp:38-78) ------------------------- */

/* op 0 = PROD, 1 = SUM (0 + sum coeff_i * x_i, in bottom order), 2 = MAX. */
void orc_eltwise(int op, int nb, const float* const* bottoms, const float* coeffs, size_t count,
                 float* top) {
  if (op == 0) {
    for (size_t i = 0; i < count; ++i) top[i] = bottoms[0][i] * bottoms[1][i];
    for (int b = 2; b < nb; ++b)
      for (size_t i = 0; i < count; ++i) top[i] = top[i] * bottoms[b][i];
  } else if (op == 1) {
    for (size_t i = 0; i < count; ++i) top[i] = 0.f;
    for (int b = 0; b < nb; ++b) {
      const float a = coeffs ? coeffs[b] : 1.f;
      for (size_t i = 0; i < count; ++i) top[i] = a * bottoms[b][i] + top[i];
    }
  } else {
    for (size_t i = 0; i < count; ++i)
      top[i] = bottoms[0][i] > bottoms[1][i] ? bottoms[0][i] : bottoms[1][i];
    for (int b = 2; b < nb; ++b)
      for (size_t i = 0; i < count; ++i)
        if (bottoms[b][i] > top[i]) top[i] = bottoms[b][i];
  }
}

/* ---- Softmax (src/layers/softmax_layer.cpp:28-63) ------------------------- */

/* Along an axis of extent `channels` with `inner` trailing elements: subtract
 * the max, expf, sum over channels in ascending order, divide. */
void orc_softmax(int outer, int channels, int inner, const float* bottom, float* top) {
  float* scale = (float*)malloc(sizeof(float) * inner);
  for (int o = 0; o < outer; ++o) {
    const float* x = bottom + (size_t)o * channels * inner;
    float* y = top + (size_t)o * channels * inner;
    for (int k = 0; k < inner; ++k) scale[k] = x[k];
    for (int c = 0; c < channels; ++c)
      for (int k = 0; k < inner; ++k)
        if (x[c * inner + k] > scale[k]) scale[k] = x[c * inner + k];
    for (int c = 0; c < channels; ++c)
      for (int k = 0; k < inner; ++k) y[c * inner + k] = expf(x[c * inner + k] + (-1.f * scale[k]));
    for (int k = 0; k < inner; ++k) scale[k] = 0.f;
    for (int c = 0; c < channels; ++c)
      for (int k = 0; k < inner; ++k) scale[k] += y[c * inner + k];
    for (int c = 0; c < channels; ++c)
      for (int k = 0; k < inner; ++k) y[c * inner + k] = y[c * inner + k] / scale[k];
  }
  free(scale);
}
