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

/* Plan for InnerProduct: top (M x N) = bottom (M x K) * W^T with W stored N x K,
 * or K x N when transpose is set (inner_product_layer.cpp:80-93; replaces the
 * caffe_gpu_gemv / caffe_gpu_gemm of inner_product_layer.cu:9-31).  It is the
 * 1x1 convolution of a [M, K, 1, 1] blob: run it with mcConvForward(num = M). */
int mcInnerProductPlanCreate(int K, int N, int transpose, mcConvPlan** plan);

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
 * reference's per-image loop.  Any batch an int can count is accepted: blobs of
 * 2^29 elements or more are processed as several runs of whole images. */
int mcConvForward(const mcConvPlan* plan, int num, const float* bottom, float* top,
                  const mcEpilogue* epilogue, void* stream);

/* mcConvForward for a plan whose output channels belong to two blobs: channels
 * [0, channels_first) of every image go to top_first [num, channels_first, Ho, Wo],
 * the others to top_second [num, Cout - channels_first, Ho, Wo].  Group 1, no
 * residual.  No counterpart in the reference: it serves two layers
 * that read the same blob with the same window (conv_layer.cu:7-22 twice) as one
 * launch over the concatenated filters. */
int mcConvForwardTwoTops(const mcConvPlan* plan, int num, const float* bottom, float* top_first,
                         int channels_first, float* top_second, const mcEpilogue* epilogue,
                         void* stream);

/* Algorithmic FLOPs of one mcConvForward call (2*MACs, padding taps counted). */
double mcConvPlanFlops(const mcConvPlan* plan, int num);

/* Name of the tile configuration the plan uses at this batch size (for reports). */
const char* mcConvPlanKernelName(const mcConvPlan* plan, int num);

/* Tuning/test knob: pin the tile configuration (index into the built-in table),
 * -1 restores the automatic choice.  No counterpart in the reference. */
int mcConvPlanForceConfig(mcConvPlan* plan, int config);

/* Tuning/test knob: pin the number of K slices a launch is cut into (the
 * slices' partial sums are added in slice order, by the last workgroup of each
 * tile to finish or, for two tops, by a second kernel, before the epilogue);
 * 0 restores the automatic choice, which slices only launches too small to
 * fill the GPU.  No counterpart in the reference. */
int mcConvPlanForceSplit(mcConvPlan* plan, int slices);

/* Tuning/test knob: a batch whose bottom or top blob reaches 2^29 elements is cut
 * into runs of whole images, one launch each (the reference loops over single
 * images, base_conv_layer.cpp:254-271, so it has no such limit); this caps a run
 * at `images` images, 0 restores the automatic choice (as many as fit).  No
 * counterpart in the reference. */
int mcConvPlanForceChunk(mcConvPlan* plan, int images);

/* A 3x3 convolution with stride 1, no dilation and one group can run as
 * F(2x2, 3x3) Winograd in one launch: the loader transforms the 4x4 input patches
 * on their way into LDS, sixteen products with the transformed filters run on the
 * matrix cores, and the output transform applies the epilogue before the store
 * (2.25 times fewer multiplications and no intermediate in memory; the sums
 * associate differently from the direct path, both within fp32 rounding of
 * conv_layer.cpp:27-42).  mode -1 lets the library decide by size, 0 keeps the
 * direct path, 1 takes this one whenever the geometry allows.
 * mcConvWinogradDefault sets the mode that plans created afterwards start with.
 * No counterpart in the reference. */
int mcConvPlanForceWinograd(mcConvPlan* plan, int mode);
int mcConvWinogradDefault(int mode);

/* Measurement hook (no counterpart in the reference): while enabled on the
 * calling thread, every contraction (one kernel launch) is bracketed by two HIP
 * events recorded on the launch stream.  mcConvTimingCollect waits for them,
 * returns the summed device time, the number of contractions and their
 * algorithmic FLOPs (those of the direct sum), and clears the list;
 * mcConvTimingCollectDetail also returns the FLOPs handed to the matrix pipe
 * (fewer on the Winograd path) and the number of Winograd contractions. */
int mcConvTimingEnable(int on);
int mcConvTimingCollect(double* total_ms, long* launches, double* flops);
int mcConvTimingCollectDetail(double* total_ms, long* launches, double* flops, double* issued_flops,
                              long* winograd);

/* Frees the calling thread's kernel scratch (the partial sums and arrival counters of
 * contractions whose channel loop is cut into slices, BatchNorm's per-part statistics):
 * grow-only device buffers, one per stream the thread has launched on, that the thread
 * owns.  They are also freed when the thread ends, and by MemPoolClear / CaffeMemPoolClear.
 * Waits for the device.  No counterpart in the reference. */
int mcReleaseScratch(void);

/* HIP stream of the calling thread's Mini-Caffe context (created on first use);
 * lets a harness record events around Net::Forward.  NULL if no device. */
void* mcCurrentStream(void);

/* ---- per-channel transforms and activations (HBM-bound) ------------------- */

/* One fused pass  v = x[o][c][i];  v -= sub[c];  v /= div[c];  v *= mul[c];
 * v += add[c];  y = act(v)  with every vector optional (NULL skips the step).
 * The step order is the reference's: BatchNorm subtracts the mean, then divides
 * by sqrt(var+eps) (batch_norm_layer.cpp:103-135); Scale multiplies, its Bias
 * adds (scale_layer.cpp:102-114, bias_layer.cpp:68-83); then ReLU / TanH /
 * Sigmoid (relu_layer.cpp:12-30, tanh_layer.cpp:14-22, sigmoid_layer.cpp:12-24).
 * Replaces ScaleForward/ScaleBiasForward (scale_layer.cu:9-25), BiasForward
 * (bias_layer.cu:9-16), ReLUForward (relu_layer.cu:8-13), TanHForward,
 * SigmoidForward and the ~10 passes of BatchNormLayer::Forward_gpu
 * (batch_norm_layer.cu:9-73).  x == y (in place) is allowed. */
typedef struct mcChannelOp {
  const float* sub;
  const float* div;
  const float* mul;
  const float* add;
  int activation;        /* enum mcActivation */
  float negative_slope;
} mcChannelOp;
int mcChannelTransform(const float* x, float* y, int outer, int channels, int inner,
                       const mcChannelOp* op, void* stream);

/* BatchNorm with stored statistics: mean[c] = blob0[c]*f, stdev[c] =
 * sqrt(blob1[c]*f + eps) with f = (blob2[0] == 0 ? 0 : 1/blob2[0])
 * (batch_norm_layer.cpp:83-90,123-126), computed on the device. */
int mcBatchNormStored(const float* blob0, const float* blob1, const float* blob2, float eps,
                      int channels, float* mean, float* stdev, void* stream);

/* BatchNorm with batch statistics (use_global_stats: false): per channel, mean
 * over num*spatial and stdev = sqrt(E[(x-mean)^2] + eps)
 * (batch_norm_layer.cpp:91-126).  Two passes over each channel's values; with few
 * channels a channel's images are cut into parts whose {mean, squared deviations}
 * are merged afterwards (the parts live in a buffer the library keeps per stream). */
int mcBatchNormBatchStats(const float* x, int num, int channels, int spatial, float eps,
                          float* mean, float* stdev, void* stream);

/* Collapses a chain of up to 4 per-channel stages (same step order as
 * mcChannelTransform, applied first to last) that follow a contraction into one
 * scale/shift pair for its epilogue:  y = acc*scale[c] + shift[c].
 * bias0 (optional) is the contraction's own bias, added before the first stage. */
int mcFoldChannelOps(const float* bias0, const mcChannelOp* stages, int num_stages, int channels,
                     float* scale, float* shift, void* stream);

/* ---- Pooling ---------------------------------------------------------------- */

enum mcPoolMethod { MC_POOL_MAX = 0, MC_POOL_AVE = 1 };

/* Output extent with Caffe's ceil rule and last-window clip
 * (pooling_layer.cpp:88-107). */
int mcPoolingOutputShape(int height, int width, int kernel_h, int kernel_w, int stride_h,
                         int stride_w, int pad_h, int pad_w, int* height_out, int* width_out);

/* bottom [planes, H, W] -> top [planes, Ho, Wo] with planes = num*channels.
 * MAX starts from -FLT_MAX over the window clipped to the image; AVE divides by
 * the window area clipped to the padded extent (pooling_layer.cpp:127-189).
 * Replaces MaxPoolForward / AvePoolForward (pooling_layer.cu:10-71). */
int mcPooling(int method, const float* bottom, float* top, int planes, int height, int width,
              int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
              void* stream);

/* ---- Eltwise ---------------------------------------------------------------- */

enum mcEltwiseOp { MC_ELT_PROD = 0, MC_ELT_SUM = 1, MC_ELT_MAX = 2 };

/* top = op over up to 8 bottoms of `count` floats; SUM is 0 + sum coeff_i*x_i in
 * bottom order (eltwise_layer.cpp:38-78); coeffs may be NULL (all 1).  An
 * activation can be fused on the result.  bottoms: host array of device
 * pointers.  Replaces MaxForward and the caffe_gpu_axpy / caffe_gpu_mul chains
 * of eltwise_layer.cu:10-50. */
int mcEltwise(int op, int num_bottoms, const float* const* bottoms, const float* coeffs,
              long count, float* top, int activation, float negative_slope, void* stream);

/* ---- Softmax ---------------------------------------------------------------- */

/* Softmax along an axis of extent `channels` with `inner` trailing elements:
 * subtract the max, expf, sum in ascending channel order, divide
 * (softmax_layer.cpp:28-63).  One launch instead of the five of
 * softmax_layer.cu:77-111. */
int mcSoftmax(const float* bottom, float* top, int outer, int channels, int inner, void* stream);

/* ---- layout ----------------------------------------------------------------- */

/* rows x width strided copy: dst[r*dst_pitch + i] = src[r*src_pitch + i].
 * Concat and Slice are one such copy per bottom/top (concat_layer.cu:8-46,
 * slice_layer.cu:8-46). */
int mcCopy2D(const float* src, long src_pitch, float* dst, long dst_pitch, long width, long rows,
             void* stream);
/* Concat of `count` sources along the axis behind `rows` leading rows, in one launch per
 * eight sources: dst[r][offset_k + i] = srcs[k][r * widths[k] + i], offsets in source
 * order, dst rows of sum(widths) floats (concat_layer.cu:8-46: one kernel per bottom
 * there).  srcs and widths are host arrays. */
int mcConcat(const float* const* srcs, const long* widths, int count, float* dst, long rows,
             void* stream);

/* Generic N-d transpose, top axis i = bottom axis order[i]
 * (permute_layer.cpp:9-106, PermuteKernel permute_layer.cu:10-28).  The
 * NCHW->NHWC order (0,2,3,1) and other "swap two adjacent axis groups" orders go
 * through an LDS-tiled transpose so both sides are coalesced. shape/order: host. */
int mcPermute(const float* bottom, float* top, int num_axes, const int* shape, const int* order,
              void* stream);

/* L2 normalisation (SSD's Normalize layer, normalize_layer.cpp:88-135; .cu:44-103).
 * across_spatial == 0: per pixel, norm = sqrt(eps + sum_c x^2); y = (x / norm) * scale.
 * across_spatial != 0: per image, norm = sqrt(sum x^2 + eps); y = (x * (1/norm)) * scale.
 * scale holds one value when channel_shared, else one per channel. */
int mcNormalize(const float* bottom, float* top, int num, int channels, int spatial,
                int across_spatial, int channel_shared, float eps, const float* scale,
                void* stream);

/* ---- detection tail (bit-exact kept indices) --------------------------------- */

/* Bytes of device scratch mcProposal needs for this problem size. */
int mcProposalWorkspaceSize(int num_proposals, int pre_nms_topn, int post_nms_topn,
                            size_t* bytes);

/* ProposalLayer::Forward (proposal_layer.cpp:261-322; device path .cu:212-276)
 * without host round trips.  All pointers are device memory.
 *   scores   [1, 2A, H, W]  (foreground = second half), bbox [1, 4A, H, W]
 *   im_info  (height, width, scale); anchors [A, 4] from GenerateAnchors (:56-85)
 *   rois     [post_nms_topn, 5] rows (0, x1, y1, x2, y2); roi_scores optional
 *   num_rois number of valid rows (device int; the caller copies it back to
 *            shape the top blob, as Forward_cpu's final Reshape does, :313-320)
 *   tie_flag optional device int: 0 when no order of equal scores had to be looked up,
 *            else 1 or 3 (see below).
 * Two steps, both queued by this call.  (1) The head of the table: the best 512
 * proposals are selected, ordered by (score descending, index ascending) and scanned;
 * the greedy pass usually reaches post_nms_topn kept boxes inside them.  Equal scores
 * among them matter only when two proposals of one score are both still alive when
 * the scan reaches them (the reference's quicksort SortBBox, :88-111, leaves equal
 * scores in an order of its own); a kernel checks that for every such group.  (2)
 * The full-size path, which skips itself on the device when step 1 settled the
 * result: all proposals are ordered by one radix sort; if equal scores reach into
 * the first pre_nms_topn + 1 places, SortBBox is replayed on the device to give the
 * same row order (tie_flag 3 = by the kernel for inputs with few equal scores, which
 * follows only the partitions that hold equal scores, 1 = by the general kernel,
 * every partition, level by level); then the overlap bit matrix and the scan. */
int mcProposal(const float* scores, const float* bbox, const float* im_info, const float* anchors,
               int A, int H, int W, int feat_stride, float min_size, int pre_nms_topn,
               int post_nms_topn, float nms_thresh, void* workspace, size_t workspace_bytes,
               float* rois, float* roi_scores, int* num_rois, int* tie_flag, void* stream);

/* The two steps of mcProposal as calls of their own, for a caller that reads num_rois
 * back anyway (the top's shape depends on it) and can read two more ints with it:
 * state[0] = tie_flag as above, state[1] = 1 when rois / num_rois are final.
 * mcProposalHead queues step 1 only (state[1] = 0: call mcProposalRest with the same
 * arguments, which starts over with the full-size path and always ends with
 * state[1] = 1).  Saves the launches of step 2 that would return at once.  No
 * counterpart in the reference. */
int mcProposalHead(const float* scores, const float* bbox, const float* im_info, const float* anchors,
                   int A, int H, int W, int feat_stride, float min_size, int pre_nms_topn,
                   int post_nms_topn, float nms_thresh, void* workspace, size_t workspace_bytes,
                   float* rois, float* roi_scores, int* num_rois, int* state, void* stream);
int mcProposalRest(const float* scores, const float* bbox, const float* im_info, const float* anchors,
                   int A, int H, int W, int feat_stride, float min_size, int pre_nms_topn,
                   int post_nms_topn, float nms_thresh, void* workspace, size_t workspace_bytes,
                   float* rois, float* roi_scores, int* num_rois, int* state, void* stream);

/* Measurement hook (no counterpart in the reference): while enabled on the calling
 * thread every mcProposal* call records HIP events between its stages on the launch
 * stream.  mcProposalTimingCollect waits for them, adds up over the calls since the
 * last collect stage_ms[0] decode + ordering of the head, [1] overlap matrix, scan and
 * check of the head + roi gather, [2] full-size path: radix sort, replay of the
 * reference's order of equal scores, gather of the best pre_nms_topn boxes, [3]
 * full-size path: NMS proper (overlap bit matrix + greedy scan) + roi gather; returns
 * the number of calls and clears the list. */
int mcProposalTimingEnable(int on);
/* Test knob (process-wide): 1 = replay the order of equal scores with the general
 * level-by-level kernel on every input, also where the kernel for inputs with few
 * equal scores would take over; 0 restores the automatic choice.  Results are the same. */
int mcProposalForceGeneralReplay(int on);
int mcProposalTimingCollect(double* stage_ms, long* calls);

/* mcProposal for callers that cannot allocate device memory or hand over a workspace
 * (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  It
 * has no counterpart in the reference.  Same arguments, results and kernels as
 * mcProposal; the scratch is an 8 MiB buffer built into the library (each GPU the
 * library runs on holds its copy until the process ends).  Problems whose scratch
 * (mcProposalWorkspaceSize) exceeds 8 MiB are refused with an error: 1 x 18 x 38 x 63
 * scores with pre_nms_topn 6000 need 6.7 MB.  The call itself allocates and frees
 * nothing.  Every call on a GPU uses that GPU's one buffer: calls that overlap on one
 * GPU (two streams, two threads) race; calls on one stream are ordered and safe.
 * The first call on a device looks the buffer's address up (hipGetSymbolAddress, which
 * may load the library's code object): make it once outside any stream capture. */
int mcProposalStatic(const float* scores, const float* bbox, const float* im_info,
                     const float* anchors, int A, int H, int W, int feat_stride, float min_size,
                     int pre_nms_topn, int post_nms_topn, float nms_thresh, float* rois,
                     float* roi_scores, int* num_rois, int* tie_flag, void* stream);

/* Bytes of device scratch mcDetectionOutput needs, and the row capacity that can
 * never be exceeded for these parameters. */
int mcDetectionOutputWorkspaceSize(int num, int num_priors, int num_classes, int share_location,
                                   int top_k, size_t* bytes);
int mcDetectionOutputMaxRows(int num, int num_priors, int num_classes, int top_k, int keep_top_k);

/* DetectionOutputLayer::Forward (detection_output_layer.cpp:74-226) on the device.
 *   loc   [num, P*loc_classes*4], conf [num, P*num_classes] (prior-major),
 *   prior [1, 2, P*4] (boxes, then variances); code_type 1 CORNER, 2 CENTER_SIZE,
 *   3 CORNER_SIZE (PriorBoxParameter.CodeType); top_k / keep_top_k -1 = unlimited;
 *   confidence_threshold -FLT_MAX = none.
 * Per image and non-background class: scores above the threshold in
 * (score desc, prior asc) order (std::stable_sort, bbox_util.cpp:523-540), cut to
 * top_k, greedy NMS with IoU <= threshold against every kept box and the adaptive
 * eta rule (:681-716); then keep_top_k per image over all classes.
 * out_rows receives [image, label, score, xmin, ymin, xmax, ymax] rows, images and
 * labels ascending, each label's boxes in NMS order; *num_rows (device int) is the
 * row count, or num rows of -1 when nothing was kept (:175-185).
 * When keep_top_k cuts an image's detections the reference re-sorts them with
 * std::sort, which leaves equal scores in an order of its own.  Here equal scores
 * at the cut are resolved by (label asc, NMS order) and a label's rows stay in NMS
 * order.  *cut_tie_flag (optional device int) reports when that could differ, as a
 * bit set over all images: 1 = the last score kept equals the first score dropped
 * (which of them survive is undefined), 2 = two kept rows of one label have equal
 * scores (their relative order is undefined); 0 = the rows are fully defined. */
int mcDetectionOutput(const float* loc, const float* conf, const float* prior, int num,
                      int num_priors, int num_classes, int share_location, int background_label,
                      int code_type, int variance_encoded_in_target, int keep_top_k,
                      float confidence_threshold, float nms_threshold, float eta, int top_k,
                      void* workspace, size_t workspace_bytes, float* out_rows, int max_rows,
                      int* num_rows, int* cut_tie_flag, void* stream);
/* Test knob (process-wide).  With a constant threshold (eta 1), at most 512 candidates
 * per class and at most 12 288 priors, the per-class work can run as three launches
 * (candidate selection, pairwise overlap bits spread over the whole chip, greedy scan)
 * followed by one launch for keep_top_k and the rows, instead of one launch per class
 * that does everything on one CU.  mode 1 (the default) takes that path where it is
 * faster (4096 priors and more), 2 wherever it fits, 0 never.  Results are the same. */
int mcDetectionOutputSplit(int mode);

/* ROIPoolingLayer::Forward (roi_pooling_layer.cpp:37-110; .cu:13-81): max pooling of
 * bottom [num, channels, height, width] over num_rois regions, rois rows of
 * [batch index, x1, y1, x2, y2] in image coordinates, top [num_rois, channels,
 * pooled_h, pooled_w].  Region ends = round(coordinate * spatial_scale), bins from
 * floor / ceil of multiples of the float bin size, clipped to the map; empty bin 0.
 * A roi with a batch index outside [0, num) (a CHECK failure in the reference's CPU
 * code) yields zeros and sets *bad_roi_flag (device int, may be NULL) to 1. */
int mcROIPooling(const float* bottom, int num, int channels, int height, int width,
                 const float* rois, int num_rois, int pooled_h, int pooled_w, float spatial_scale,
                 float* top, int* bad_roi_flag, void* stream);

/* PSROIPoolingLayer::Forward (psroi_pooling_layer.cpp:45-122; .cu:13-89): position-
 * sensitive average pooling, bottom [num, output_dim*group_size^2, height, width],
 * top [num_rois, output_dim, group_size, group_size]; bin (ph, pw) of output channel
 * c averages input channel (c*group_size + ph)*group_size + pw.  Region corners are
 * rounded before scaling, the end corner as round(x2 + 1) (the CPU code's form), the
 * region is at least 0.1 wide; sums run row-major over the bin; empty bin 0. */
int mcPSROIPooling(const float* bottom, int num, int output_dim, int group_size, int height,
                   int width, const float* rois, int num_rois, float spatial_scale, float* top,
                   int* bad_roi_flag, void* stream);

/* ---- further layers of the model zoo ------------------------------------------ */

/* Elementwise functions with up to three scalar parameters; bottom == top allowed.
 *   MC_UNARY_POWER      (p1 + p0*x)^p2           power_layer.cpp:17-40, .cu:8-29
 *   MC_UNARY_EXP        p1 * exp(p0*x)           exp_layer.cpp:31-45  (p0 = log(base)*scale,
 *                                                p1 = base^shift, both folded by the caller)
 *   MC_UNARY_LOG        p2 * log(p1 + p0*x)      log_layer.cpp:35-54  (p2 = 1/log(base))
 *   MC_UNARY_ABS        |x|                      absval_layer.cpp:8-13
 *   MC_UNARY_BNLL       log(1 + exp(x))          bnll_layer.cpp:8-18
 *   MC_UNARY_ELU        max(x,0)+p0*(exp(min(x,0))-1)   elu_layer.cpp:8-18
 *   MC_UNARY_THRESHOLD  x > p0 ? 1 : 0           threshold_layer.cpp:13-21 */
enum mcUnaryOp {
  MC_UNARY_POWER = 0,
  MC_UNARY_EXP = 1,
  MC_UNARY_LOG = 2,
  MC_UNARY_ABS = 3,
  MC_UNARY_BNLL = 4,
  MC_UNARY_ELU = 5,
  MC_UNARY_THRESHOLD = 6
};
int mcUnary(int op, const float* bottom, float* top, long count, float p0, float p1, float p2,
            void* stream);

/* PReLULayer::Forward (prelu_layer.cpp:50-84; .cu:9-33): max(x,0) + slope[c]*min(x,0)
 * with c the index on the `channels` axis of a [outer, channels, inner] view, or 0
 * when channel_shared.  bottom == top allowed. */
int mcPReLU(const float* bottom, float* top, int outer, int channels, int inner,
            const float* slope, int channel_shared, void* stream);

/* LRNLayer::CrossChannelForward (lrn_layer.cpp:112-155; .cu:9-94):
 * top = bottom * (k + alpha/local_size * sum of squares over local_size neighbouring
 * channels)^-beta, the window centred on the channel and clipped to the blob. */
int mcLRNAcrossChannels(const float* bottom, float* top, int num, int channels, int height,
                        int width, int local_size, float alpha, float beta, float k,
                        void* stream);

/* LRNLayer::WithinChannelForward (lrn_layer.cpp:20-66,157-164: Split -> Power(2) ->
 * average Pooling(local_size, pad (local_size-1)/2) -> Power(1 + alpha*., -beta) ->
 * Eltwise PROD) as one pass over `planes` maps of height x width. */
int mcLRNWithinChannel(const float* bottom, float* top, long planes, int height, int width,
                       int local_size, float alpha, float beta, void* stream);

/* ArgMaxLayer::Forward_cpu (argmax_layer.cpp:56-93; the reference has no device
 * version): the top_k largest of the `dim` values of every line of a
 * [outer, dim, inner] view, in the order of std::greater on (value, index) pairs —
 * among equal values the larger index comes first.  Indices are stored as floats.
 *   MC_ARGMAX_INDEX             top[outer, top_k, inner] = index
 *   MC_ARGMAX_VALUE             top[outer, top_k, inner] = value
 *   MC_ARGMAX_INDEX_THEN_VALUE  top[outer, 2, top_k] = indices then values (inner == 1) */
enum mcArgMaxLayout { MC_ARGMAX_INDEX = 0, MC_ARGMAX_VALUE = 1, MC_ARGMAX_INDEX_THEN_VALUE = 2 };
int mcArgMax(const float* bottom, float* top, long outer, int dim, int inner, int top_k,
             int layout, void* stream);

/* ReductionLayer::Forward (reduction_layer.cpp:38-72; .cu:8-40): top[i] = coeff *
 * reduce(bottom[i, 0:dim]); MEAN divides by dim.  Values as in ReductionParameter. */
enum mcReduceOp { MC_REDUCE_SUM = 1, MC_REDUCE_ASUM = 2, MC_REDUCE_SUMSQ = 3, MC_REDUCE_MEAN = 4 };
int mcReduction(int op, const float* bottom, float* top, int num, int dim, float coeff,
                void* stream);

/* MVNLayer::Forward (mvn_layer.cpp:36-75; .cu:8-49): per row of a [num, dim] view,
 * x - mean, divided by sqrt(mean((x-mean)^2)) + eps when normalize_variance. */
int mcMVN(const float* bottom, float* top, int num, int dim, int normalize_variance, float eps,
          void* stream);

/* top[r, :] = table[(int)rows[r], :] (+ bias).  EmbedLayer::Forward
 * (embed_layer.cpp:62-79; .cu:9-35) with the row numbers held as floats, and the
 * row copy of FilterLayer::Forward (filter_layer.cpp:61-75).  A row number outside
 * [0, table_rows) (a DCHECK in the reference) yields NaN. */
int mcGatherRows(const float* table, int table_rows, int row_len, const float* rows, long num_rows,
                 const float* bias, float* top, void* stream);

/* CropLayer::Forward (crop_layer.cpp:61-107; .cu:11-80): top = the box of shape
 * top_shape at `offsets` inside bottom; up to MC_MAX_AXES axes. */
#define MC_MAX_AXES 8
int mcCrop(const float* bottom, float* top, int num_axes, const int* bottom_shape,
           const int* top_shape, const int* offsets, void* stream);

/* TileLayer::Forward (tile_layer.cpp:24-35; .cu:9-29): [outer, inner] -> [outer, tiles, inner]. */
int mcTile(const float* bottom, float* top, long outer, int inner, int tiles, void* stream);

/* Fill `count` floats with `value` (caffe_gpu_set, math_functions.cu:70-82). */
int mcFill(float* dst, long count, float value, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* MCHIP_KERNELS_H_ */
