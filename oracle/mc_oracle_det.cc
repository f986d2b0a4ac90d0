/*
 * mc_oracle_det.cc — CPU restatement of Mini-Caffe's detection tail
 * (Normalize, PriorBox, Proposal, DetectionOutput) and of the two region
 * pooling layers that consume Proposal's rois (ROIPooling, PSROIPooling).
 *
 * TEST INFRASTRUCTURE ONLY (see mc_oracle.c).  C++ rather than C because the
 * reference's orderings are those of std::stable_sort and std::sort; using the
 * same library routines reproduces them, ties included.
 *
 * Floating point: the reference's expressions are kept operand for operand.
 * Two of its files call exp() unqualified with only <cmath> in scope
 * (src/layers/proposal_layer.cpp:30-31, src/util/bbox_util.cpp:281-292); that
 * resolves to ::exp(double), so the product with the width is formed in double
 * and narrowed on assignment.  Whether a generated protobuf header would pull
 * <math.h> in and select expf instead cannot be checked here: PARITY UNPINNED
 * for that one choice (the two readings differ in the last float bit).  The
 * "/ 2." literals promote to double as written.
 * Build flags keep a*b+c as two roundings (-ffp-contract=off, no -march).
 *
 * How each function is pinned (tests/test_oracle_det.py):
 *   anchors            the published py-faster-rcnn table for base 16
 *   proposal decode    closed form in float64 on boxes away from clip edges
 *   SortBBox           descending order on tie-free data; partial-sort contract;
 *                      the order of EQUAL scores by seven literal vectors whose
 *                      expected order was traced by hand from the reference text
 *                      (a changed comparison or recursion cut fails one of them)
 *   NMS (both)         brute force: kept set is independent and maximal w.r.t.
 *                      "earlier kept box overlaps > thr"
 *   prior box          SSD300 prior count 8732 and closed-form centres / sizes
 *   detection output   float64 walk on <= 96 priors: all three code types, variance in
 *                      the prior or in the target, shared and per-class locations,
 *                      any background label, adaptive eta threshold, keep_top_k.
 *                      Not pinned: std::sort's order of equal scores at the
 *                      keep_top_k cut (PARITY UNPINNED for that tie case)
 *   normalize          closed form
 *   roi / psroi pool   special cases that reduce to numpy routines: a roi over the
 *                      whole map with 1x1 bins is the global max / mean, with one
 *                      bin per cell the identity; integer-aligned rois are block
 *                      max / block mean of a reshaped array; empty bins give 0
 */
#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstring>
#include <map>
#include <utility>
#include <vector>

extern "C" {

/* ---- Normalize (src/layers/normalize_layer.cpp:88-135) -------------------- */

void orc_normalize(int num, int channels, int spatial, const float* bottom, const float* scale,
                   int across_spatial, int channel_shared, float eps, float* top) {
  const int dim = channels * spatial;
  std::vector<float> norm(spatial);
  for (int n = 0; n < num; ++n) {
    const float* x = bottom + (size_t)n * dim;
    float* y = top + (size_t)n * dim;
    if (across_spatial) {
      float asum = 0.f;  // caffe_cpu_asum of the squares
      for (int i = 0; i < dim; ++i) asum += std::fabs(x[i] * x[i]);
      const float nrm = std::pow(asum + eps, 0.5f);
      const float inv = static_cast<float>(1.0 / nrm);
      for (int i = 0; i < dim; ++i) y[i] = inv * x[i];
    } else {
      for (int s = 0; s < spatial; ++s) norm[s] = eps;
      for (int c = 0; c < channels; ++c)
        for (int s = 0; s < spatial; ++s) norm[s] += x[c * spatial + s] * x[c * spatial + s];
      for (int s = 0; s < spatial; ++s) norm[s] = std::pow(norm[s], 0.5f);
      for (int c = 0; c < channels; ++c)
        for (int s = 0; s < spatial; ++s) y[c * spatial + s] = x[c * spatial + s] / norm[s];
    }
    if (channel_shared) {
      for (int i = 0; i < dim; ++i) y[i] *= scale[0];
    } else {
      for (int c = 0; c < channels; ++c)
        for (int s = 0; s < spatial; ++s) y[c * spatial + s] = y[c * spatial + s] * scale[c];
    }
  }
}

/* ---- PriorBox (src/layers/prior_box_layer.cpp:116-217) -------------------- */

/* aspect_ratios: the de-duplicated, flipped list the layer builds in LayerSetUp
 * (first entry 1).  variance: 1 or 4 values.  out: 2 * dim floats. */
void orc_prior_box(int layer_h, int layer_w, int img_h, int img_w, const float* min_sizes, int n_min,
                   const float* max_sizes, int n_max, const float* aspect_ratios, int n_ar,
                   const float* variance, int n_var, int clip, float step_h_in, float step_w_in,
                   float offset, float* out) {
  float step_w, step_h;
  if (step_w_in == 0 || step_h_in == 0) {
    step_w = static_cast<float>(img_w) / layer_w;
    step_h = static_cast<float>(img_h) / layer_h;
  } else {
    step_w = step_w_in;
    step_h = step_h_in;
  }
  const int num_priors = n_ar * n_min + n_max;
  const int dim = layer_h * layer_w * num_priors * 4;
  int idx = 0;
  for (int h = 0; h < layer_h; ++h) {
    for (int w = 0; w < layer_w; ++w) {
      float center_x = (w + offset) * step_w;
      float center_y = (h + offset) * step_h;
      float box_width, box_height;
      for (int s = 0; s < n_min; ++s) {
        int min_size_ = min_sizes[s];
        box_width = box_height = min_size_;
        out[idx++] = (center_x - box_width / 2.) / img_w;
        out[idx++] = (center_y - box_height / 2.) / img_h;
        out[idx++] = (center_x + box_width / 2.) / img_w;
        out[idx++] = (center_y + box_height / 2.) / img_h;
        if (n_max > 0) {
          int max_size_ = max_sizes[s];
          box_width = box_height = sqrt(min_size_ * max_size_);
          out[idx++] = (center_x - box_width / 2.) / img_w;
          out[idx++] = (center_y - box_height / 2.) / img_h;
          out[idx++] = (center_x + box_width / 2.) / img_w;
          out[idx++] = (center_y + box_height / 2.) / img_h;
        }
        for (int r = 0; r < n_ar; ++r) {
          float ar = aspect_ratios[r];
          if (fabs(ar - 1.) < 1e-6) continue;
          box_width = min_size_ * sqrtf(ar);
          box_height = min_size_ / sqrtf(ar);
          out[idx++] = (center_x - box_width / 2.) / img_w;
          out[idx++] = (center_y - box_height / 2.) / img_h;
          out[idx++] = (center_x + box_width / 2.) / img_w;
          out[idx++] = (center_y + box_height / 2.) / img_h;
        }
      }
    }
  }
  if (clip)
    for (int d = 0; d < dim; ++d) out[d] = std::min<float>(std::max<float>(out[d], 0.), 1.);
  float* var = out + dim;
  if (n_var == 1) {
    for (int d = 0; d < dim; ++d) var[d] = variance[0];
  } else {
    for (int d = 0; d < dim; ++d) var[d] = variance[d % 4];
  }
}

/* ---- Proposal (src/layers/proposal_layer.cpp:14-322) ---------------------- */

/* GenerateAnchors (:56-85): ratio-major, scale-minor. */
void orc_generate_anchors(int base_size, const float* ratios, int nr, const float* scales, int ns,
                          float* anchors) {
  const float base_area = static_cast<float>(base_size * base_size);
  const float center = static_cast<float>(0.5 * (base_size - 1));
  for (int i = 0; i < nr; ++i) {
    const float ratio_w = static_cast<float>(round(std::sqrt(base_area / ratios[i])));
    const float ratio_h = static_cast<float>(round(ratio_w * ratios[i]));
    for (int j = 0; j < ns; ++j) {
      const float scale_w = 0.5f * static_cast<float>(ratio_w * scales[j] - 1);
      const float scale_h = 0.5f * static_cast<float>(ratio_h * scales[j] - 1);
      anchors[0] = center - scale_w;
      anchors[1] = center - scale_h;
      anchors[2] = center + scale_w;
      anchors[3] = center + scale_h;
      anchors += 4;
    }
  }
}

/* TransformBBox (:14-53). */
static int transform_box(float* box, float dx, float dy, float d_log_w, float d_log_h,
                         float img_width, float img_height, float min_bbox_size) {
  const float w = box[2] - box[0] + 1;
  const float h = box[3] - box[1] + 1;
  const float ctr_x = box[0] + 0.5f * w;
  const float ctr_y = box[1] + 0.5f * h;
  const float pred_ctr_x = dx * w + ctr_x;
  const float pred_ctr_y = dy * h + ctr_y;
  const float pred_w = ::exp(static_cast<double>(d_log_w)) * w;
  const float pred_h = ::exp(static_cast<double>(d_log_h)) * h;
  box[0] = pred_ctr_x - 0.5f * pred_w;
  box[1] = pred_ctr_y - 0.5f * pred_h;
  box[2] = pred_ctr_x + 0.5f * pred_w;
  box[3] = pred_ctr_y + 0.5f * pred_h;
  box[0] = std::max(0.f, std::min(box[0], img_width - 1));
  box[1] = std::max(0.f, std::min(box[1], img_height - 1));
  box[2] = std::max(0.f, std::min(box[2], img_width - 1));
  box[3] = std::max(0.f, std::min(box[3], img_height - 1));
  const float box_w = box[2] - box[0] + 1;
  const float box_h = box[3] - box[1] + 1;
  return (box_w >= min_bbox_size) && (box_h >= min_bbox_size);
}

/* GenerateProposalsCPU (:114-148): order h, w, anchor; score is the foreground
 * map (second half of bottom[0]) times the min-size mask. */
void orc_generate_proposals(const float* fg_scores, const float* bbox, const float* anchors, int A,
                            int H, int W, float img_h, float img_w, float min_bbox_size,
                            int feat_stride, float* proposals) {
  const int fm = H * W;
  float* p = proposals;
  for (int h = 0; h < H; ++h)
    for (int w = 0; w < W; ++w) {
      const float x = w * feat_stride;
      const float y = h * feat_stride;
      const float* box = bbox + h * W + w;
      const float* score = fg_scores + h * W + w;
      for (int k = 0; k < A; ++k) {
        p[0] = x + anchors[k * 4 + 0];
        p[1] = y + anchors[k * 4 + 1];
        p[2] = x + anchors[k * 4 + 2];
        p[3] = y + anchors[k * 4 + 3];
        p[4] = transform_box(p, box[(k * 4 + 0) * fm], box[(k * 4 + 1) * fm], box[(k * 4 + 2) * fm],
                             box[(k * 4 + 3) * fm], img_w, img_h, min_bbox_size) *
               score[k * fm];
        p += 5;
      }
    }
}

/* SortBBox (:88-111): quicksort on rows of 5 floats by column 4, descending,
 * first element as pivot, moving rows through a hole; the part right of a pivot
 * is only sorted while it starts before num_top. */
static void sort_rows(float* rois, int left, int right, int num_top) {
  int first = left, last = right;
  float key[5];
  memcpy(key, rois + 5 * first, sizeof(key));
  while (first < last) {
    while (first < last && rois[last * 5 + 4] <= key[4]) last--;
    memcpy(rois + 5 * first, rois + 5 * last, sizeof(key));
    while (first < last && rois[first * 5 + 4] >= key[4]) first++;
    memcpy(rois + 5 * last, rois + 5 * first, sizeof(key));
  }
  memcpy(rois + 5 * first, key, sizeof(key));
  if (left < first - 1) sort_rows(rois, left, first - 1, num_top);
  if (first + 1 < num_top && first + 1 < right) sort_rows(rois, first + 1, right, num_top);
}

void orc_sort_bbox(float* rois, int n, int num_top) {
  if (n > 0) sort_rows(rois, 0, n - 1, num_top);
}

/* NonMaximumSuppressionCPU (:150-185): +1 pixel areas, ov > thr suppresses,
 * stops once max_rois boxes are kept. */
int orc_nms_pixel(int n, const float* proposals, float thr, int max_rois, int* kept) {
  std::vector<float> areas(n);
  for (int i = 0; i < n; ++i) {
    const float* p = proposals + i * 5;
    areas[i] = (p[2] - p[0] + 1) * (p[3] - p[1] + 1);
  }
  std::vector<char> removed(n, 0);
  int count = 0;
  for (int i = 0; i < n; ++i) {
    if (removed[i]) continue;
    removed[i] = 1;
    kept[count++] = i;
    if (count == max_rois) break;
    for (int j = i + 1; j < n; ++j) {
      const float* p1 = proposals + i * 5;
      const float* p2 = proposals + j * 5;
      const float x1 = std::max(p1[0], p2[0]);
      const float y1 = std::max(p1[1], p2[1]);
      const float x2 = std::min(p1[2], p2[2]);
      const float y2 = std::min(p1[3], p2[3]);
      const float w = std::max(0.f, x2 - x1 + 1);
      const float h = std::max(0.f, y2 - y1 + 1);
      const float area = w * h;
      const float ov = area / (areas[i] + areas[j] - area);
      if (ov > thr) removed[j] = 1;
    }
  }
  return count;
}

/* ProposalLayer::Forward_cpu (:261-322).  scores: bottom[0] (2A x H x W, batch 1),
 * bbox: bottom[1] (4A x H x W), im_info: (height, width, scale).
 * sorted_out (optional): the num_proposals x 5 table after SortBBox.
 * Returns the number of rois; rois is R x 5 with batch index 0. */
int orc_proposal(const float* scores, const float* bbox, const float* im_info, int A, int H, int W,
                 const float* anchors, int feat_stride, int min_size, int pre_nms_topn,
                 int post_nms_topn, float nms_thresh, float* rois, float* roi_scores,
                 int* kept_indices, float* sorted_out) {
  const int n = A * H * W;
  const float min_bbox_size = min_size * im_info[2];
  const int pre = std::min(n, pre_nms_topn);
  std::vector<float> props((size_t)n * 5);
  orc_generate_proposals(scores + n, bbox, anchors, A, H, W, im_info[0], im_info[1], min_bbox_size,
                         feat_stride, props.data());
  orc_sort_bbox(props.data(), n, pre);
  std::vector<int> kept(post_nms_topn);
  const int r = orc_nms_pixel(pre, props.data(), nms_thresh, post_nms_topn, kept.data());
  for (int i = 0; i < r; ++i) {
    const float* p = props.data() + kept[i] * 5;
    rois[i * 5 + 0] = 0;
    rois[i * 5 + 1] = p[0];
    rois[i * 5 + 2] = p[1];
    rois[i * 5 + 3] = p[2];
    rois[i * 5 + 4] = p[3];
    if (roi_scores) roi_scores[i] = p[4];
    if (kept_indices) kept_indices[i] = kept[i];
  }
  if (sorted_out) memcpy(sorted_out, props.data(), sizeof(float) * props.size());
  return r;
}

/* ---- DetectionOutput (src/layers/detection_output_layer.cpp:74-226,
 *      src/util/bbox_util.cpp) ------------------------------------------------ */

struct Box {
  float xmin, ymin, xmax, ymax, size;
};

/* BBoxSize (bbox_util.cpp:80-97) for a box without a cached size. */
static float box_size(const Box& b) {
  if (b.xmax < b.xmin || b.ymax < b.ymin) return 0;
  const float width = b.xmax - b.xmin;
  const float height = b.ymax - b.ymin;
  return width * height;
}

/* DecodeBBox (bbox_util.cpp:242-330). code_type: 1 CORNER, 2 CENTER_SIZE, 3 CORNER_SIZE. */
static void decode_box(const float* prior, const float* var, int code_type, int var_in_target,
                       int clip, const float* loc, Box* out) {
  const float pxmin = prior[0], pymin = prior[1], pxmax = prior[2], pymax = prior[3];
  if (code_type == 1) {
    if (var_in_target) {
      out->xmin = pxmin + loc[0];
      out->ymin = pymin + loc[1];
      out->xmax = pxmax + loc[2];
      out->ymax = pymax + loc[3];
    } else {
      out->xmin = pxmin + var[0] * loc[0];
      out->ymin = pymin + var[1] * loc[1];
      out->xmax = pxmax + var[2] * loc[2];
      out->ymax = pymax + var[3] * loc[3];
    }
  } else if (code_type == 2) {
    float prior_width = pxmax - pxmin;
    float prior_height = pymax - pymin;
    float prior_center_x = (pxmin + pxmax) / 2.;
    float prior_center_y = (pymin + pymax) / 2.;
    float cx, cy, w, h;
    if (var_in_target) {
      cx = loc[0] * prior_width + prior_center_x;
      cy = loc[1] * prior_height + prior_center_y;
      w = ::exp(static_cast<double>(loc[2])) * prior_width;
      h = ::exp(static_cast<double>(loc[3])) * prior_height;
    } else {
      cx = var[0] * loc[0] * prior_width + prior_center_x;
      cy = var[1] * loc[1] * prior_height + prior_center_y;
      w = ::exp(static_cast<double>(var[2] * loc[2])) * prior_width;
      h = ::exp(static_cast<double>(var[3] * loc[3])) * prior_height;
    }
    out->xmin = cx - w / 2.;
    out->ymin = cy - h / 2.;
    out->xmax = cx + w / 2.;
    out->ymax = cy + h / 2.;
  } else {
    float prior_width = pxmax - pxmin;
    float prior_height = pymax - pymin;
    if (var_in_target) {
      out->xmin = pxmin + loc[0] * prior_width;
      out->ymin = pymin + loc[1] * prior_height;
      out->xmax = pxmax + loc[2] * prior_width;
      out->ymax = pymax + loc[3] * prior_height;
    } else {
      out->xmin = pxmin + var[0] * loc[0] * prior_width;
      out->ymin = pymin + var[1] * loc[1] * prior_height;
      out->xmax = pxmax + var[2] * loc[2] * prior_width;
      out->ymax = pymax + var[3] * loc[3] * prior_height;
    }
  }
  out->size = box_size(*out);
  if (clip) {
    out->xmin = std::max(std::min(out->xmin, 1.f), 0.f);
    out->ymin = std::max(std::min(out->ymin, 1.f), 0.f);
    out->xmax = std::max(std::min(out->xmax, 1.f), 0.f);
    out->ymax = std::max(std::min(out->ymax, 1.f), 0.f);
    out->size = box_size(*out);
  }
}

/* JaccardOverlap (bbox_util.cpp:184-204) on normalised boxes with cached sizes. */
static float jaccard(const Box& a, const Box& b) {
  Box in;
  if (b.xmin > a.xmax || b.xmax < a.xmin || b.ymin > a.ymax || b.ymax < a.ymin) {
    in.xmin = in.ymin = in.xmax = in.ymax = 0;
  } else {
    in.xmin = std::max(a.xmin, b.xmin);
    in.ymin = std::max(a.ymin, b.ymin);
    in.xmax = std::min(a.xmax, b.xmax);
    in.ymax = std::min(a.ymax, b.ymax);
  }
  const float iw = in.xmax - in.xmin, ih = in.ymax - in.ymin;
  if (iw > 0 && ih > 0) {
    const float isz = iw * ih;
    return isz / (a.size + b.size - isz);
  }
  return 0.;
}

static bool score_desc(const std::pair<float, int>& a, const std::pair<float, int>& b) {
  return a.first > b.first;
}
static bool score_desc2(const std::pair<float, std::pair<int, int> >& a,
                        const std::pair<float, std::pair<int, int> >& b) {
  return a.first > b.first;
}

/* ApplyNMSFast (bbox_util.cpp:681-716) with GetMaxScoreIndex (:523-540). */
static void nms_fast(const std::vector<Box>& boxes, const float* scores, int stride, int n,
                     float score_thr, float nms_thr, float eta, int top_k, std::vector<int>* keep) {
  std::vector<std::pair<float, int> > cand;
  for (int i = 0; i < n; ++i)
    if (scores[(size_t)i * stride] > score_thr) cand.push_back(std::make_pair(scores[(size_t)i * stride], i));
  std::stable_sort(cand.begin(), cand.end(), score_desc);
  if (top_k > -1 && top_k < static_cast<int>(cand.size())) cand.resize(top_k);
  float adaptive = nms_thr;
  keep->clear();
  for (size_t c = 0; c < cand.size(); ++c) {
    const int idx = cand[c].second;
    bool ok = true;
    for (size_t k = 0; k < keep->size() && ok; ++k) ok = jaccard(boxes[idx], boxes[(*keep)[k]]) <= adaptive;
    if (ok) keep->push_back(idx);
    if (ok && eta < 1 && adaptive > 0.5) adaptive *= eta;
  }
}

/* DetectionOutputLayer::Forward_cpu.  loc: num x (P*loc_classes*4); conf: num x
 * (P*num_classes), prior-major; prior: 2 x (P*4).  out receives rows of 7 floats
 * (capacity max_rows); returns the number of rows (num rows of -1 when nothing
 * is kept, as :175-185), -1 when out is too small, -2 where the reference aborts. */
int orc_detection_output(const float* loc, const float* conf, const float* prior, int num,
                         int num_priors, int num_classes, int share_location, int background_label,
                         int code_type, int var_in_target, int keep_top_k, float conf_thr,
                         float nms_thr, float eta, int top_k, float* out, int max_rows) {
  const int loc_classes = share_location ? 1 : num_classes;
  /* Shared locations carry the label -1; with background_label_id == -1 DecodeBBoxesAll
   * (bbox_util.cpp:366-371) skips them as "background" and the layer then dies with
   * "Could not find location predictions for label -1" (detection_output_layer.cpp:122-126). */
  if (share_location && background_label == -1) return -2;
  std::vector<std::map<int, std::vector<int> > > all_indices(num);
  std::vector<std::vector<std::vector<Box> > > decoded(num);
  int num_kept = 0;
  for (int i = 0; i < num; ++i) {
    decoded[i].resize(loc_classes);
    for (int c = 0; c < loc_classes; ++c) {
      const int label = share_location ? -1 : c;
      if (label == background_label) continue;
      decoded[i][c].resize(num_priors);
      for (int p = 0; p < num_priors; ++p)
        decode_box(prior + p * 4, prior + (num_priors + p) * 4, code_type, var_in_target, 0,
                   loc + ((size_t)i * num_priors + p) * loc_classes * 4 + c * 4, &decoded[i][c][p]);
    }
    std::map<int, std::vector<int> > indices;
    int num_det = 0;
    const float* conf_i = conf + (size_t)i * num_priors * num_classes;
    for (int c = 0; c < num_classes; ++c) {
      if (c == background_label) continue;
      const std::vector<Box>& boxes = decoded[i][share_location ? 0 : c];
      nms_fast(boxes, conf_i + c, num_classes, num_priors, conf_thr, nms_thr, eta, top_k, &indices[c]);
      num_det += static_cast<int>(indices[c].size());
    }
    if (keep_top_k > -1 && num_det > keep_top_k) {
      std::vector<std::pair<float, std::pair<int, int> > > pairs;
      for (auto& kv : indices)
        for (int idx : kv.second)
          pairs.push_back(std::make_pair(conf_i[(size_t)idx * num_classes + kv.first],
                                         std::make_pair(kv.first, idx)));
      std::sort(pairs.begin(), pairs.end(), score_desc2);
      pairs.resize(keep_top_k);
      std::map<int, std::vector<int> > fresh;
      for (auto& p : pairs) fresh[p.second.first].push_back(p.second.second);
      all_indices[i] = fresh;
      num_kept += keep_top_k;
    } else {
      all_indices[i] = indices;
      num_kept += num_det;
    }
  }
  if (num_kept == 0) {
    for (int i = 0; i < num && i < max_rows; ++i) {
      for (int k = 0; k < 7; ++k) out[i * 7 + k] = -1;
      out[i * 7] = i;
    }
    return num;
  }
  int count = 0;
  for (int i = 0; i < num; ++i) {
    const float* conf_i = conf + (size_t)i * num_priors * num_classes;
    for (auto& kv : all_indices[i]) {
      const int label = kv.first;
      const std::vector<Box>& boxes = decoded[i][share_location ? 0 : label];
      for (int idx : kv.second) {
        if (count >= max_rows) return -1;
        float* row = out + (size_t)count * 7;
        row[0] = i;
        row[1] = label;
        row[2] = conf_i[(size_t)idx * num_classes + label];
        row[3] = boxes[idx].xmin;
        row[4] = boxes[idx].ymin;
        row[5] = boxes[idx].xmax;
        row[6] = boxes[idx].ymax;
        ++count;
      }
    }
  }
  return count;
}

/* ---- ROIPooling (src/layers/roi_pooling_layer.cpp:37-110) -------------------
 * rois: R rows [batch index, x1, y1, x2, y2] in image coordinates.  Region ends
 * are rounded after scaling; bins use floor / ceil of multiples of the float bin
 * size, are shifted by the region start and clipped to the map; an empty bin
 * yields 0, otherwise the maximum (initial value -FLT_MAX).  The reference
 * CHECK-fails on a batch index outside [0, num); here such a roi returns -1. */
int orc_roi_pooling(const float* bottom, int num, int channels, int height, int width,
                    const float* rois, int num_rois, int pooled_h, int pooled_w,
                    float spatial_scale, float* top) {
  for (int n = 0; n < num_rois; ++n) {
    const float* roi = rois + 5 * n;
    const int batch = static_cast<int>(roi[0]);
    if (batch < 0 || batch >= num) return -1;
    const int roi_start_w = static_cast<int>(round(roi[1] * spatial_scale));
    const int roi_start_h = static_cast<int>(round(roi[2] * spatial_scale));
    const int roi_end_w = static_cast<int>(round(roi[3] * spatial_scale));
    const int roi_end_h = static_cast<int>(round(roi[4] * spatial_scale));
    const int roi_height = std::max(roi_end_h - roi_start_h + 1, 1);
    const int roi_width = std::max(roi_end_w - roi_start_w + 1, 1);
    const float bin_size_h = static_cast<float>(roi_height) / static_cast<float>(pooled_h);
    const float bin_size_w = static_cast<float>(roi_width) / static_cast<float>(pooled_w);
    for (int c = 0; c < channels; ++c) {
      const float* plane = bottom + (static_cast<size_t>(batch) * channels + c) * height * width;
      float* out = top + (static_cast<size_t>(n) * channels + c) * pooled_h * pooled_w;
      for (int ph = 0; ph < pooled_h; ++ph) {
        for (int pw = 0; pw < pooled_w; ++pw) {
          int hstart = static_cast<int>(std::floor(static_cast<float>(ph) * bin_size_h));
          int wstart = static_cast<int>(std::floor(static_cast<float>(pw) * bin_size_w));
          int hend = static_cast<int>(std::ceil(static_cast<float>(ph + 1) * bin_size_h));
          int wend = static_cast<int>(std::ceil(static_cast<float>(pw + 1) * bin_size_w));
          hstart = std::min(std::max(hstart + roi_start_h, 0), height);
          hend = std::min(std::max(hend + roi_start_h, 0), height);
          wstart = std::min(std::max(wstart + roi_start_w, 0), width);
          wend = std::min(std::max(wend + roi_start_w, 0), width);
          const bool is_empty = (hend <= hstart) || (wend <= wstart);
          float v = is_empty ? 0.f : -FLT_MAX;
          for (int h = hstart; h < hend; ++h)
            for (int w = wstart; w < wend; ++w) v = std::max(v, plane[h * width + w]);
          out[ph * pooled_w + pw] = v;
        }
      }
    }
  }
  return 0;
}

/* ---- PSROIPooling (src/layers/psroi_pooling_layer.cpp:45-122) ---------------
 * Position-sensitive average pooling: output channel c, bin (ph, pw) averages
 * input channel (c*group + ph)*group + pw over the bin.  Region corners are
 * rounded BEFORE scaling (end corner: round(x2 + 1)), the region is at least
 * 0.1 wide, bins use floor / ceil of float positions, clipped to the map; the
 * sum runs row-major over the bin and is divided by the bin area; an empty bin
 * yields 0. */
int orc_psroi_pooling(const float* bottom, int num, int output_dim, int group_size, int height,
                      int width, const float* rois, int num_rois, float spatial_scale,
                      float* top) {
  const int pooled_h = group_size, pooled_w = group_size;
  const int channels = output_dim * group_size * group_size;
  for (int n = 0; n < num_rois; ++n) {
    const float* roi = rois + 5 * n;
    const int batch = static_cast<int>(roi[0]);
    if (batch < 0 || batch >= num) return -1;
    const float roi_start_w = static_cast<float>(round(roi[1]) * spatial_scale);
    const float roi_start_h = static_cast<float>(round(roi[2]) * spatial_scale);
    const float roi_end_w = static_cast<float>(round(roi[3] + 1) * spatial_scale);
    const float roi_end_h = static_cast<float>(round(roi[4] + 1) * spatial_scale);
    const float roi_height = std::max(roi_end_h - roi_start_h, static_cast<float>(0.1));
    const float roi_width = std::max(roi_end_w - roi_start_w, static_cast<float>(0.1));
    const float bin_size_h = roi_height / static_cast<float>(pooled_h);
    const float bin_size_w = roi_width / static_cast<float>(pooled_w);
    const float* batch_data = bottom + static_cast<size_t>(batch) * channels * height * width;
    for (int c = 0; c < output_dim; ++c) {
      float* out = top + (static_cast<size_t>(n) * output_dim + c) * pooled_h * pooled_w;
      for (int ph = 0; ph < pooled_h; ++ph) {
        for (int pw = 0; pw < pooled_w; ++pw) {
          int hstart = static_cast<int>(std::floor(static_cast<float>(ph) * bin_size_h + roi_start_h));
          int wstart = static_cast<int>(std::floor(static_cast<float>(pw) * bin_size_w + roi_start_w));
          int hend = static_cast<int>(std::ceil(static_cast<float>(ph + 1) * bin_size_h + roi_start_h));
          int wend = static_cast<int>(std::ceil(static_cast<float>(pw + 1) * bin_size_w + roi_start_w));
          hstart = std::min(std::max(hstart, 0), height);
          hend = std::min(std::max(hend, 0), height);
          wstart = std::min(std::max(wstart, 0), width);
          wend = std::min(std::max(wend, 0), width);
          const bool is_empty = (hend <= hstart) || (wend <= wstart);
          const int fm_c = (c * group_size + ph) * group_size + pw;
          const float* fm = batch_data + static_cast<size_t>(fm_c) * height * width;
          float out_sum = 0;
          for (int h = hstart; h < hend; ++h)
            for (int w = wstart; w < wend; ++w) out_sum += fm[h * width + w];
          const int bin_area = (hend - hstart) * (wend - wstart);
          out[ph * pooled_w + pw] = is_empty ? 0.f : out_sum / static_cast<float>(bin_area);
        }
      }
    }
  }
  return 0;
}

}  // extern "C"
