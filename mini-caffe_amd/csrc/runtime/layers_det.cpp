// Detection-tail layers: Proposal (registered as "Proposal", type() reports
// "ProposalLayer" like the reference) and DetectionOutput.
#include <algorithm>
#include <cfloat>
#include <cmath>

#include "layer.hpp"

namespace caffe {

// ---------------------------------------------------------------------------
// Proposal (reference src/layers/proposal_layer.cpp:56-85,205-322; .cu:212-276)
// ---------------------------------------------------------------------------
class ProposalLayer : public Layer {
 public:
  explicit ProposalLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "ProposalLayer"; }
  bool ShapesTopInForward() const override { return true; }
  int ExactNumBottomBlobs() const override { return 3; }
  int MinTopBlobs() const override { return 1; }
  int MaxTopBlobs() const override { return 2; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("proposal_param");
    base_size_ = static_cast<int>(p.get_int("base_size", 16));
    feat_stride_ = static_cast<int>(p.get_int("feat_stride", 16));
    pre_nms_topn_ = static_cast<int>(p.get_int("pre_nms_topn", 6000));
    post_nms_topn_ = static_cast<int>(p.get_int("post_nms_topn", 300));
    nms_thresh_ = static_cast<float>(p.get_float("nms_thresh", 0.7));
    min_size_ = static_cast<int>(p.get_int("min_size", 16));
    CHECK_GT(pre_nms_topn_, 0);
    CHECK_GT(post_nms_topn_, 0);
    vector<float> ratios, scales;
    for (int i = 0; i < p.count("ratio"); ++i) ratios.push_back(static_cast<float>(p.get_float("ratio", 0., i)));
    for (int i = 0; i < p.count("scale"); ++i) scales.push_back(static_cast<float>(p.get_float("scale", 0., i)));
    if (ratios.empty()) ratios = {0.5f, 1.f, 2.f};    // caffe.proto defaults
    if (scales.empty()) scales = {8.f, 16.f, 32.f};
    anchors_.Reshape(vector<int>{static_cast<int>(ratios.size() * scales.size()), 4});
    GenerateAnchors(ratios, scales);
    Reshape(bottom, top);
  }

  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    top[0]->Reshape(vector<int>{bottom[0]->shape(0) * post_nms_topn_, 5});
    if (top.size() > 1) top[1]->Reshape(vector<int>{bottom[0]->shape(0) * post_nms_topn_});
  }

 protected:
  // Ratio-major, scale-minor anchor table around a base_size square
  // (proposal_layer.cpp:56-85); float/double mix as there.
  void GenerateAnchors(const vector<float>& ratios, const vector<float>& scales) {
    const float base_area = static_cast<float>(base_size_ * base_size_);
    const float center = static_cast<float>(0.5 * (base_size_ - 1));
    real_t* a = anchors_.mutable_cpu_data();
    for (size_t i = 0; i < ratios.size(); ++i) {
      const float ratio_w = static_cast<float>(round(std::sqrt(base_area / ratios[i])));
      const float ratio_h = static_cast<float>(round(ratio_w * ratios[i]));
      for (size_t j = 0; j < scales.size(); ++j) {
        const float scale_w = 0.5f * static_cast<float>(ratio_w * scales[j] - 1);
        const float scale_h = 0.5f * static_cast<float>(ratio_h * scales[j] - 1);
        a[0] = center - scale_w;
        a[1] = center - scale_h;
        a[2] = center + scale_w;
        a[3] = center + scale_h;
        a += 4;
      }
    }
  }

  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_EQ(bottom[0]->shape(0), 1) << "Only support single scale.";
    const int A = anchors_.shape(0);
    CHECK_EQ(bottom[0]->shape(1), 2 * A) << "score blob must have 2 x num_anchors channels";
    CHECK_EQ(bottom[1]->shape(1), 4 * A) << "bbox blob must have 4 x num_anchors channels";
    CHECK_GE(bottom[2]->count(), 3) << "im_info needs (height, width, scale)";
    const int H = bottom[0]->height(), W = bottom[0]->width();
    const int n = A * H * W;
    size_t bytes = 0;
    MC_CHECK(mcProposalWorkspaceSize(n, pre_nms_topn_, post_nms_topn_, &bytes));
    workspace_.Reshape(vector<int>{static_cast<int>((bytes + 3) / 4)});
    counters_.Reshape(vector<int>{3});
    // full-size tops while the kernels run; shrunk to the roi count afterwards
    top[0]->Reshape(vector<int>{post_nms_topn_, 5});
    if (top.size() > 1) top[1]->Reshape(vector<int>{post_nms_topn_});
    // The top's shape depends on the data (proposal_layer.cpp:313-320), so the roi count
    // has to come back to the host; with it comes the word that says whether the head of
    // the proposal table settled the result.  Only if it did not is the full-size path
    // queued (counters: roi count, equal-score replay flag, result final).
    int num_rois = 0;
    for (int step = 0; step < 2; ++step) {
      int* counters = counters_.mutable_gpu_data();
      MC_CHECK((step == 0 ? mcProposalHead : mcProposalRest)(
          bottom[0]->gpu_data(), bottom[1]->gpu_data(), bottom[2]->gpu_data(), anchors_.gpu_data(), A,
          H, W, feat_stride_, static_cast<float>(min_size_), pre_nms_topn_, post_nms_topn_,
          nms_thresh_, workspace_.mutable_gpu_data(), bytes, top[0]->mutable_gpu_data(),
          top.size() > 1 ? top[1]->mutable_gpu_data() : nullptr, counters, counters + 1,
          cur_stream()));
      const int* host = counters_.cpu_data();
      num_rois = host[0];
      if (host[2] != 0) break;
    }
    top[0]->Reshape(vector<int>{num_rois, 5});
    if (top.size() > 1) top[1]->Reshape(vector<int>{num_rois});
  }

  int base_size_ = 16, feat_stride_ = 16, pre_nms_topn_ = 6000, post_nms_topn_ = 300, min_size_ = 16;
  float nms_thresh_ = 0.7f;
  Blob anchors_, workspace_;
  BlobInt counters_;
};
REGISTER_LAYER_CLASS(Proposal);

// ---------------------------------------------------------------------------
// DetectionOutput (reference src/layers/detection_output_layer.cpp:11-226; .cu:14-152)
// ---------------------------------------------------------------------------
class DetectionOutputLayer : public Layer {
 public:
  explicit DetectionOutputLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "DetectionOutput"; }
  bool ShapesTopInForward() const override { return true; }
  int ExactNumBottomBlobs() const override { return 3; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("detection_output_param");
    CHECK(p.has("num_classes")) << "Must specify num_classes";
    num_classes_ = static_cast<int>(p.get_int("num_classes"));
    share_location_ = p.get_bool("share_location", true);
    background_label_id_ = static_cast<int>(p.get_int("background_label_id", 0));
    const string code = p.get_string("code_type", "CORNER");
    if (code == "CORNER" || code == "1") code_type_ = 1;
    else if (code == "CENTER_SIZE" || code == "2") code_type_ = 2;
    else if (code == "CORNER_SIZE" || code == "3") code_type_ = 3;
    else LOG(FATAL) << "Unknown LocLossType.";
    variance_encoded_in_target_ = p.get_bool("variance_encoded_in_target", false);
    keep_top_k_ = static_cast<int>(p.get_int("keep_top_k", -1));
    confidence_threshold_ = p.has("confidence_threshold")
                                ? static_cast<float>(p.get_float("confidence_threshold"))
                                : -FLT_MAX;
    const Message& nms = p.sub("nms_param");
    nms_threshold_ = static_cast<float>(nms.get_float("nms_threshold", 0.3));
    CHECK_GE(nms_threshold_, 0.) << "nms_threshold must be non negative.";
    eta_ = static_cast<float>(nms.get_float("eta", 1.0));
    CHECK_GT(eta_, 0.);
    CHECK_LE(eta_, 1.);
    top_k_ = nms.has("top_k") ? static_cast<int>(nms.get_int("top_k")) : -1;
  }

  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_EQ(bottom[0]->num(), bottom[1]->num());
    num_priors_ = bottom[2]->height() / 4;
    const int loc_classes = share_location_ ? 1 : num_classes_;
    CHECK_EQ(num_priors_ * loc_classes * 4, bottom[0]->channels())
        << "Number of priors must match number of location predictions.";
    CHECK_EQ(num_priors_ * num_classes_, bottom[1]->channels())
        << "Number of priors must match number of confidence predictions.";
    // the number of kept boxes is unknown before NMS: one placeholder row
    top[0]->Reshape(vector<int>{1, 7});
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const int num = bottom[0]->num();
    size_t bytes = 0;
    MC_CHECK(mcDetectionOutputWorkspaceSize(num, num_priors_, num_classes_, share_location_ ? 1 : 0,
                                            top_k_, &bytes));
    CHECK_LT(bytes / 4, static_cast<size_t>(INT_MAX)) << "DetectionOutput workspace too large";
    workspace_.Reshape(vector<int>{static_cast<int>((bytes + 3) / 4)});
    const int max_rows =
        mcDetectionOutputMaxRows(num, num_priors_, num_classes_, top_k_, keep_top_k_);
    CHECK_LT(static_cast<long>(max_rows) * 7, static_cast<long>(INT_MAX));
    counter_.Reshape(vector<int>{1});
    top[0]->Reshape(vector<int>{max_rows, 7});
    MC_CHECK(mcDetectionOutput(bottom[0]->gpu_data(), bottom[1]->gpu_data(), bottom[2]->gpu_data(),
                               num, num_priors_, num_classes_, share_location_ ? 1 : 0,
                               background_label_id_, code_type_,
                               variance_encoded_in_target_ ? 1 : 0, keep_top_k_,
                               confidence_threshold_, nms_threshold_, eta_, top_k_,
                               workspace_.mutable_gpu_data(), bytes, top[0]->mutable_gpu_data(),
                               max_rows, counter_.mutable_gpu_data(), nullptr, cur_stream()));
    // data-dependent top shape (detection_output_layer.cpp:166-189)
    const int rows = counter_.cpu_data()[0];
    top[0]->Reshape(vector<int>{rows, 7});
  }

  int num_classes_ = 0, background_label_id_ = 0, code_type_ = 1, keep_top_k_ = -1, top_k_ = -1;
  int num_priors_ = 0;
  bool share_location_ = true, variance_encoded_in_target_ = false;
  float confidence_threshold_ = -FLT_MAX, nms_threshold_ = 0.3f, eta_ = 1.f;
  Blob workspace_;
  BlobInt counter_;
};
REGISTER_LAYER_CLASS(DetectionOutput);

// ---------------------------------------------------------------------------
// ROIPooling (reference src/layers/roi_pooling_layer.cpp:15-110; .cu:13-81) and
// PSROIPooling (psroi_pooling_layer.cpp:18-122; .cu:13-89): the consumers of
// Proposal's rois.  As in the reference the top keeps the row count the rois blob
// had at Reshape time; Forward pools the rows the rois blob has then (Proposal
// shrinks it to the kept count) and the remaining rows hold the reference's fill
// value (-FLT_MAX for ROIPooling, 0 for PSROIPooling).
// ---------------------------------------------------------------------------
class RegionPoolingBase : public Layer {
 public:
  explicit RegionPoolingBase(const LayerParameter& param) : Layer(param) {}
  int ExactNumBottomBlobs() const override { return 2; }
  int ExactNumTopBlobs() const override { return 1; }

 protected:
  // rois rows to pool now, and the fill of the rows beyond them
  int PrepareRows(const vector<Blob*>& bottom, const vector<Blob*>& top, float fill) {
    CHECK_EQ(bottom[1]->count(1), 5) << "rois must be rows of [batch index, x1, y1, x2, y2]";
    const int rows = std::min(bottom[1]->shape(0), top[0]->shape(0));
    const long per_row = top[0]->count(1);
    const long rest = (top[0]->shape(0) - rows) * per_row;
    if (rest > 0)
      MC_CHECK(mcFill(top[0]->mutable_gpu_data() + rows * per_row, rest, fill, cur_stream()));
    return rows;
  }
  float spatial_scale_ = 1.f;
};

class ROIPoolingLayer : public RegionPoolingBase {
 public:
  explicit ROIPoolingLayer(const LayerParameter& param) : RegionPoolingBase(param) {}
  const char* type() const override { return "ROIPooling"; }
  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("roi_pooling_param");
    pooled_h_ = static_cast<int>(p.get_int("pooled_h", 0));
    pooled_w_ = static_cast<int>(p.get_int("pooled_w", 0));
    CHECK_GT(pooled_h_, 0) << "pooled_h must be > 0";
    CHECK_GT(pooled_w_, 0) << "pooled_w must be > 0";
    spatial_scale_ = static_cast<float>(p.get_float("spatial_scale", 1.));
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_EQ(bottom[0]->num_axes(), 4) << "ROIPooling bottom must be num x channels x height x width";
    top[0]->Reshape(vector<int>{bottom[1]->shape(0), bottom[0]->shape(1), pooled_h_, pooled_w_});
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const int rows = PrepareRows(bottom, top, -FLT_MAX);
    MC_CHECK(mcROIPooling(bottom[0]->gpu_data(), bottom[0]->shape(0), bottom[0]->shape(1),
                          bottom[0]->shape(2), bottom[0]->shape(3), bottom[1]->gpu_data(), rows,
                          pooled_h_, pooled_w_, spatial_scale_,
                          rows ? top[0]->mutable_gpu_data() : nullptr, nullptr, cur_stream()));
  }
  int pooled_h_ = 0, pooled_w_ = 0;
};
REGISTER_LAYER_CLASS(ROIPooling);

class PSROIPoolingLayer : public RegionPoolingBase {
 public:
  explicit PSROIPoolingLayer(const LayerParameter& param) : RegionPoolingBase(param) {}
  const char* type() const override { return "PSROIPooling"; }
  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("psroi_pooling_param");
    CHECK(p.has("spatial_scale") && p.has("output_dim") && p.has("group_size"))
        << "psroi_pooling_param needs spatial_scale, output_dim and group_size";
    spatial_scale_ = static_cast<float>(p.get_float("spatial_scale", 1.));
    output_dim_ = static_cast<int>(p.get_int("output_dim", 0));
    group_size_ = static_cast<int>(p.get_int("group_size", 0));
    CHECK_GT(output_dim_, 0) << "output_dim must be > 0";
    CHECK_GT(group_size_, 0) << "group_size must be > 0";
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_EQ(bottom[0]->num_axes(), 4) << "PSROIPooling bottom must be num x channels x height x width";
    CHECK_EQ(bottom[0]->shape(1), output_dim_ * group_size_ * group_size_)
        << "input channel number does not match layer parameters";
    top[0]->Reshape(vector<int>{bottom[1]->shape(0), output_dim_, group_size_, group_size_});
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const int rows = PrepareRows(bottom, top, 0.f);
    MC_CHECK(mcPSROIPooling(bottom[0]->gpu_data(), bottom[0]->shape(0), output_dim_, group_size_,
                            bottom[0]->shape(2), bottom[0]->shape(3), bottom[1]->gpu_data(), rows,
                            spatial_scale_, rows ? top[0]->mutable_gpu_data() : nullptr, nullptr,
                            cur_stream()));
  }
  int output_dim_ = 0, group_size_ = 0;
};
REGISTER_LAYER_CLASS(PSROIPooling);

}  // namespace caffe
