/*
 * mchip/kernels.h — C ABI of the gfx950 device kernels behind Mini-Caffe's
 * Layer::Forward_gpu.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void*; NULL = the null stream).  Nothing here allocates per call
 * except the explicit *Create functions.  All functions return 0 on success
 * and a non-zero code on failure; mcLastError() then holds a message for the
 * calling thread.  Blob layout is the reference's: contiguous row-major NCHW,
 * offset = ((n*C + c)*H + h)*W + w  (reference include/caffe/blob.hpp:155-158),
 * element type float (reference include/caffe/base.hpp:48).
 *
 * Each declaration names the reference function it stands in for.
 */
#ifndef MCHIP_KERNELS_H_
#define MCHIP_KERNELS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- errors --------------------------------------------------------------- */

/* Message of the last failure on the calling thread ("" if none).
 * Plays the role of CUDA_CHECK -> caffe::Error (reference src/common.hpp:23-28). */
const char* mcLastError(void);

/* ---- dense contraction: Convolution / Deconvolution / InnerProduct ------- */

/* Geometry of one 2-D (de)convolution, in the reference's terms
 * (reference src/layers/base_conv_layer.cpp:11-252). */
typedef struct mcConvGeom {
  int channels_in;   /* bottom channels                                   */
  int height_in;     /* bottom H                                          */
  int width_in;      /* bottom W                                          */
  int channels_out;  /* num_output                                        */
  int kernel_h, kernel_w;
  int stride_h, stride_w;
  int pad_h, pad_w;
  int dilation_h, dilation_w;
  int group;
  int transposed;    /* 0 = Convolution, 1 = Deconvolution                */
} mcConvGeom;

/* Activation applied by the fused epilogue. */
enum mcActivation {
  MC_ACT_NONE = 0,
  MC_ACT_RELU = 1,    /* x>0 ? x : slope*x  (reference relu_layer.cpp:12-30) */
  MC_ACT_TANH = 2,    /* reference tanh_layer.cpp:14-22                      */
  MC_ACT_SIGMOID = 3  /* reference sigmoid_layer.cpp                         */
};

/* Per-output-channel epilogue  y = act((acc * scale[c] + shift[c]) + residual).
 * scale == NULL means 1, shift == NULL means 0, residual == NULL means none.
 * Folds forward_cpu_bias (base_conv_layer.cpp:273-278), BatchNorm
 * (batch_norm_layer.cpp:103-135), Scale (scale_layer.cpp:102-118), Eltwise SUM
 * (eltwise_layer.cpp:50-58) and the activation into the contraction kernel. */
typedef struct mcEpilogue {
  const float* scale;     /* [channels_out] device, or NULL */
  const float* shift;     /* [channels_out] device, or NULL */
  const float* residual;  /* same shape as the output, device, or NULL */
  int activation;         /* enum mcActivation */
  float negative_slope;   /* for MC_ACT_RELU */
} mcEpilogue;

typedef struct mcConvPlan mcConvPlan;

/* Builds the tap tables for an implicit-GEMM (de)convolution and allocates the
 * device copy of the filter in the kernel's K-major layout.  Replaces the
 * col_buffer_ / im2col set-up of BaseConvolutionLayer::Reshape
 * (base_conv_layer.cpp:227-239): no column buffer exists here. */
int mcConvPlanCreate(const mcConvGeom* geom, mcConvPlan** plan);
int mcConvPlanDestroy(mcConvPlan* plan);

/* Output height/width for this geometry (conv_layer.cpp:12-25,
 * deconv_layer.cpp:11-25). */
int mcConvPlanOutputShape(const mcConvPlan* plan, int* height_out, int* width_out);

/* (Re)packs the filter blob.  weights: device pointer in the reference's
 * layout, [Cout, Cin/g, kh, kw] for Convolution and [Cin, Cout/g, kh, kw] for
 * Deconvolution (base_conv_layer.cpp:124-139).  Call again when weights change. */
int mcConvPlanSetWeights(mcConvPlan* plan, const float* weights, void* stream);

/* Whole-batch forward: bottom [num, Cin, H, W] -> top [num, Cout, Ho, Wo].
 * Replaces ConvolutionLayer::Forward_gpu (conv_layer.cu:7-22) and
 * DeconvolutionLayer::Forward_gpu (deconv_layer.cu:7-22) including the bias
 * add; the batch is folded into the GEMM column dimension instead of the
 * reference's per-image loop. */
int mcConvForward(const mcConvPlan* plan, int num, const float* bottom, float* top,
                  const mcEpilogue* epilogue, void* stream);

/* Algorithmic FLOPs of one mcConvForward call (2*MACs, padding taps counted). */
double mcConvPlanFlops(const mcConvPlan* plan, int num);

/* Name of the tile configuration the plan uses at this batch size (for reports). */
const char* mcConvPlanKernelName(const mcConvPlan* plan, int num);

/* Tuning/test knob: pin the tile configuration (index into the built-in table),
 * -1 restores the automatic choice.  No counterpart in the reference. */
int mcConvPlanForceConfig(mcConvPlan* plan, int config);

#ifdef __cplusplus
}
#endif

#endif /* MCHIP_KERNELS_H_ */
