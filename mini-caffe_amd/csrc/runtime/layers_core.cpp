// Layers of the dense path: Input, Convolution, Deconvolution, InnerProduct,
// BatchNorm, Scale, Bias, ReLU, TanH, Sigmoid, Pooling, Eltwise, Softmax.
//
// Host-side set-up and shape inference restate the reference layer of the same
// name (file:line given per class); Forward_gpu hands device pointers to the
// kernel ABI in mchip/kernels.h on the calling thread's stream.
#include <algorithm>
#include <cmath>

#include "layer.hpp"

namespace caffe {

// ---------------------------------------------------------------------------
// Input (reference src/layers/input_layer.cpp:7-21)
// ---------------------------------------------------------------------------
class InputLayer : public Layer {
 public:
  explicit InputLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Input"; }
  int ExactNumBottomBlobs() const override { return 0; }
  int MinTopBlobs() const override { return 1; }
  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("input_param");
    const int num_top = static_cast<int>(top.size());
    const int num_shape = p.count("shape");
    CHECK(num_shape == 0 || num_shape == 1 || num_shape == num_top)
        << "Must specify 'shape' once, once per top blob, or not at all: " << num_top
        << " tops vs. " << num_shape << " shapes.";
    for (int i = 0; num_shape > 0 && i < num_top; ++i) {
      const Message& s = p.sub("shape", num_shape == 1 ? 0 : i);
      vector<int> shape;
      for (int d = 0; d < s.count("dim"); ++d) shape.push_back(static_cast<int>(s.get_int("dim", 0, d)));
      top[i]->Reshape(shape);
    }
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {}

 protected:
  void Forward_cpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {}
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {}
};
REGISTER_LAYER_CLASS(Input);

// ---------------------------------------------------------------------------
// Shared by the three contraction layers: folding of following channel stages
// into the kernel epilogue.
// ---------------------------------------------------------------------------
class ContractionLayer : public Layer {
 public:
  explicit ContractionLayer(const LayerParameter& param) : Layer(param), plan_(nullptr) {}
  ~ContractionLayer() override {
    if (plan_) mcConvPlanDestroy(plan_);
  }
  bool AcceptsEpilogue() const override { return true; }
  int MaxAffineFollowers() const override { return 4; }
  void SetEpilogue(const vector<Layer*>& followers) override {
    followers_ = followers;
    fold_version_ = ~0ull;
    residual_ = nullptr;
    residual_act_ = nullptr;
  }
  bool AcceptsResidual() const override {
    for (Layer* f : followers_) {
      const string ty = f->type();
      if (ty == "ReLU" || ty == "TanH" || ty == "Sigmoid") return false;
    }
    return true;
  }
  void SetResidual(Blob* residual, Layer* activation) override {
    residual_ = residual;
    residual_act_ = activation;
  }

 protected:
  // Builds the epilogue for `channels` output channels with optional own bias.
  void PrepareEpilogue(int channels, const shared_ptr<Blob>& bias, mcEpilogue* ep) {
    ep->scale = nullptr;
    ep->shift = nullptr;
    ep->residual = nullptr;
    ep->activation = MC_ACT_NONE;
    ep->negative_slope = 0.f;
    vector<mcChannelOp> stages;
    uint64_t version = BlobVersion(bias) * 1000003ull + followers_.size();
    for (Layer* f : followers_) version = version * 1000003ull + f->ChannelStageVersion();
    const bool refold = version != fold_version_ || fold_channels_ != channels;
    int n_affine = 0;
    for (Layer* f : followers_) {
      mcChannelOp op = {nullptr, nullptr, nullptr, nullptr, MC_ACT_NONE, 0.f};
      const string ty = f->type();
      const bool is_act = ty == "ReLU" || ty == "TanH" || ty == "Sigmoid";
      if (is_act || refold) f->GetChannelStage(&op);
      if (is_act) {
        ep->activation = op.activation;
        ep->negative_slope = op.negative_slope;
      } else {
        ++n_affine;
        stages.push_back(op);
      }
    }
    if (residual_) {
      ep->residual = residual_->gpu_data();
      if (residual_act_) {
        mcChannelOp op = {nullptr, nullptr, nullptr, nullptr, MC_ACT_NONE, 0.f};
        residual_act_->GetChannelStage(&op);
        ep->activation = op.activation;
        ep->negative_slope = op.negative_slope;
      }
    }
    if (n_affine == 0) {
      // Plain bias add keeps the reference's rounding: acc + bias[c].
      if (bias) ep->shift = bias->gpu_data();
      return;
    }
    if (refold) {
      fold_scale_.Reshape(vector<int>{channels});
      fold_shift_.Reshape(vector<int>{channels});
      MC_CHECK(mcFoldChannelOps(bias ? bias->gpu_data() : nullptr, stages.data(),
                                static_cast<int>(stages.size()), channels,
                                fold_scale_.mutable_gpu_data(), fold_shift_.mutable_gpu_data(),
                                cur_stream()));
      fold_version_ = version;
      fold_channels_ = channels;
    }
    ep->scale = fold_scale_.gpu_data();
    ep->shift = fold_shift_.gpu_data();
  }

  // Re-packs the filter when its blob was written since the last forward.
  void SyncWeights() {
    const uint64_t v = BlobVersion(blobs_[0]);
    if (v != weights_version_) {
      MC_CHECK(mcConvPlanSetWeights(plan_, blobs_[0]->gpu_data(), cur_stream()));
      weights_version_ = v;
    }
  }

  mcConvPlan* plan_;
  uint64_t weights_version_ = ~0ull;
  vector<Layer*> followers_;
  Blob* residual_ = nullptr;       // added after the per-channel stages
  Layer* residual_act_ = nullptr;  // activation applied after the residual
  Blob fold_scale_, fold_shift_;
  uint64_t fold_version_ = ~0ull;
  int fold_channels_ = -1;
};

// ---------------------------------------------------------------------------
// Convolution / Deconvolution
// (reference src/layers/base_conv_layer.cpp:11-252, conv_layer.cpp:12-42,
//  deconv_layer.cpp:11-42; device path conv_layer.cu:7-22, deconv_layer.cu:7-22)
// ---------------------------------------------------------------------------
class BaseConvolutionLayer : public ContractionLayer {
 public:
  explicit BaseConvolutionLayer(const LayerParameter& param) : ContractionLayer(param) {}
  int MinBottomBlobs() const override { return 1; }
  int MinTopBlobs() const override { return 1; }
  bool EqualNumBottomTopBlobs() const override { return true; }
  bool AcceptsEpilogue() const override { return true; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("convolution_param");
    CHECK(!p.get_bool("force_nd_im2col", false)) << "force_nd_im2col is not supported";
    const int channel_axis = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("axis", 1)));
    CHECK_EQ(channel_axis, 1) << "only axis = 1 convolutions are supported";
    CHECK_EQ(bottom[0]->num_axes(), 4) << "only 2-D convolution is supported "
                                       << "(bottom must be num x channels x height x width)";
    auto pair = [&](const char* rep, const char* h, const char* w, int def, int* oh, int* ow) {
      if (p.has(h) || p.has(w)) {
        CHECK_EQ(0, p.count(rep)) << "Either " << rep << " or " << h << "/" << w
                                  << " should be specified; not both.";
        *oh = static_cast<int>(p.get_int(h, def));
        *ow = static_cast<int>(p.get_int(w, def));
      } else {
        const int n = p.count(rep);
        CHECK(n == 0 || n == 1 || n == 2)
            << rep << " must be specified once, or once per spatial dimension (" << rep
            << " specified " << n << " times; 2 spatial dims).";
        *oh = n == 0 ? def : static_cast<int>(p.get_int(rep, def, 0));
        *ow = n == 0 ? def : static_cast<int>(p.get_int(rep, def, n == 1 ? 0 : 1));
      }
    };
    CHECK(p.has("kernel_size") || p.has("kernel_h") || p.has("kernel_w"))
        << "kernel_size must be specified once, or once per spatial dimension "
        << "(kernel_size specified 0 times; 2 spatial dims).";
    pair("kernel_size", "kernel_h", "kernel_w", 0, &geom_.kernel_h, &geom_.kernel_w);
    CHECK_GT(geom_.kernel_h, 0) << "Filter dimensions must be nonzero.";
    CHECK_GT(geom_.kernel_w, 0) << "Filter dimensions must be nonzero.";
    pair("stride", "stride_h", "stride_w", 1, &geom_.stride_h, &geom_.stride_w);
    CHECK_GT(geom_.stride_h, 0) << "Stride dimensions must be nonzero.";
    CHECK_GT(geom_.stride_w, 0) << "Stride dimensions must be nonzero.";
    pair("pad", "pad_h", "pad_w", 0, &geom_.pad_h, &geom_.pad_w);
    {
      const int n = p.count("dilation");
      CHECK(n == 0 || n == 1 || n == 2) << "dilation must be specified once, or once per "
                                        << "spatial dimension";
      geom_.dilation_h = n == 0 ? 1 : static_cast<int>(p.get_int("dilation", 1, 0));
      geom_.dilation_w = n == 0 ? 1 : static_cast<int>(p.get_int("dilation", 1, n == 1 ? 0 : 1));
    }
    geom_.channels_in = bottom[0]->shape(1);
    if (depthwise()) {
      // One filter per input channel whatever num_output and group say.
      geom_.channels_out = geom_.channels_in;
      geom_.group = geom_.channels_in;
    } else {
      geom_.channels_out = static_cast<int>(p.get_int("num_output", 0));
      CHECK_GT(geom_.channels_out, 0);
      geom_.group = static_cast<int>(p.get_int("group", 1));
    }
    CHECK_EQ(geom_.channels_in % geom_.group, 0);
    CHECK_EQ(geom_.channels_out % geom_.group, 0) << "Number of output should be multiples of group.";
    geom_.transposed = transposed() ? 1 : 0;
    // blobs_[0]: filters, blobs_[1]: biases (optional)
    vector<int> weight_shape;
    if (!transposed()) {
      weight_shape = {geom_.channels_out, geom_.channels_in / geom_.group, geom_.kernel_h,
                      geom_.kernel_w};
    } else {
      weight_shape = {geom_.channels_in, geom_.channels_out / geom_.group, geom_.kernel_h,
                      geom_.kernel_w};
    }
    bias_term_ = p.get_bool("bias_term", true);
    vector<int> bias_shape(bias_term_ ? 1 : 0, geom_.channels_out);
    if (!blobs_.empty()) {
      CHECK_EQ(static_cast<size_t>(1 + bias_term_), blobs_.size()) << "Incorrect number of weight blobs.";
      if (weight_shape != blobs_[0]->shape()) {
        Blob expected(weight_shape);
        LOG(FATAL) << "Incorrect weight shape: expected shape " << expected.shape_string()
                   << "; instead, shape was " << blobs_[0]->shape_string();
      }
      if (bias_term_ && bias_shape != blobs_[1]->shape()) {
        Blob expected(bias_shape);
        LOG(FATAL) << "Incorrect bias shape: expected shape " << expected.shape_string()
                   << "; instead, shape was " << blobs_[1]->shape_string();
      }
    } else {
      blobs_.resize(bias_term_ ? 2 : 1);
      blobs_[0].reset(new Blob(weight_shape));
      FillConstant(p.sub("weight_filler"), blobs_[0].get());
      if (bias_term_) {
        blobs_[1].reset(new Blob(bias_shape));
        FillConstant(p.sub("bias_filler"), blobs_[1].get());
      }
    }
  }

  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_EQ(bottom[0]->num_axes(), 4) << "bottom num_axes may not change.";
    CHECK_EQ(bottom[0]->shape(1), geom_.channels_in)
        << "Input size incompatible with convolution kernel.";
    for (size_t i = 1; i < bottom.size(); ++i)
      CHECK(bottom[0]->shape() == bottom[i]->shape()) << "All inputs must have the same shape.";
    geom_.height_in = bottom[0]->shape(2);
    geom_.width_in = bottom[0]->shape(3);
    const int eh = geom_.dilation_h * (geom_.kernel_h - 1) + 1;
    const int ew = geom_.dilation_w * (geom_.kernel_w - 1) + 1;
    int ho, wo;
    if (!transposed()) {
      ho = (geom_.height_in + 2 * geom_.pad_h - eh) / geom_.stride_h + 1;
      wo = (geom_.width_in + 2 * geom_.pad_w - ew) / geom_.stride_w + 1;
    } else {
      ho = geom_.stride_h * (geom_.height_in - 1) + eh - 2 * geom_.pad_h;
      wo = geom_.stride_w * (geom_.width_in - 1) + ew - 2 * geom_.pad_w;
    }
    for (Blob* t : top) t->Reshape(vector<int>{bottom[0]->shape(0), geom_.channels_out, ho, wo});
  }

 protected:
  virtual bool transposed() const = 0;
  virtual bool depthwise() const { return false; }

  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (!plan_ || plan_h_ != geom_.height_in || plan_w_ != geom_.width_in) {
      if (plan_) mcConvPlanDestroy(plan_);
      plan_ = nullptr;
      MC_CHECK(mcConvPlanCreate(&geom_, &plan_));
      plan_h_ = geom_.height_in;
      plan_w_ = geom_.width_in;
      weights_version_ = ~0ull;
    }
    SyncWeights();
    mcEpilogue ep;
    PrepareEpilogue(geom_.channels_out, bias_term_ ? blobs_[1] : shared_ptr<Blob>(), &ep);
    for (size_t i = 0; i < bottom.size(); ++i) {
      MC_CHECK(mcConvForward(plan_, bottom[i]->shape(0), bottom[i]->gpu_data(),
                             top[i]->mutable_gpu_data(), &ep, cur_stream()));
    }
  }

  mcConvGeom geom_ = {};
  bool bias_term_ = true;
  int plan_h_ = -1, plan_w_ = -1;
};

class ConvolutionLayer : public BaseConvolutionLayer {
 public:
  explicit ConvolutionLayer(const LayerParameter& param) : BaseConvolutionLayer(param) {}
  ~ConvolutionLayer() override {
    if (merged_plan_) mcConvPlanDestroy(merged_plan_);
  }
  const char* type() const override { return "Convolution"; }

  // ---- sibling merge: this layer and an adopted one as a single launch --------
  bool SiblingKey(vector<int>* key) const override {
    if (geom_.group != 1 || !followers_.empty() || residual_ != nullptr) return false;
    *key = {geom_.channels_in, geom_.kernel_h, geom_.kernel_w, geom_.stride_h, geom_.stride_w,
            geom_.pad_h,       geom_.pad_w,    geom_.dilation_h, geom_.dilation_w};
    return true;
  }
  void AdoptSibling(Layer* sibling, Blob* sibling_top) override {
    sibling_ = static_cast<ConvolutionLayer*>(sibling);
    sibling_top_ = sibling_top;
    merged_version_ = ~0ull;
  }

 protected:
  bool transposed() const override { return false; }

  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (!sibling_ || bottom.size() != 1) {
      BaseConvolutionLayer::Forward_gpu(bottom, top);
      return;
    }
    // One contraction over both layers' filters; the kernel stores each layer's
    // channels into that layer's top.
    const int m1 = geom_.channels_out, m2 = sibling_->geom_.channels_out;
    mcConvGeom g = geom_;
    g.channels_out = m1 + m2;
    if (!merged_plan_ || merged_h_ != g.height_in || merged_w_in_ != g.width_in || merged_m_ != m1 + m2) {
      if (merged_plan_) mcConvPlanDestroy(merged_plan_);
      merged_plan_ = nullptr;
      MC_CHECK(mcConvPlanCreate(&g, &merged_plan_));
      merged_h_ = g.height_in;
      merged_w_in_ = g.width_in;
      merged_m_ = m1 + m2;
      merged_version_ = ~0ull;
    }
    const bool any_bias = bias_term_ || sibling_->bias_term_;
    uint64_t v = BlobVersion(blobs_[0]) * 1000003ull + BlobVersion(sibling_->blobs_[0]);
    if (bias_term_) v = v * 1000003ull + BlobVersion(blobs_[1]);
    if (sibling_->bias_term_) v = v * 1000003ull + BlobVersion(sibling_->blobs_[1]);
    if (v != merged_version_) {
      const long w1 = blobs_[0]->count(), w2 = sibling_->blobs_[0]->count();
      merged_filter_.Reshape(vector<int>{m1 + m2, geom_.channels_in, geom_.kernel_h, geom_.kernel_w});
      float* w = merged_filter_.mutable_gpu_data();
      MC_CHECK(mcCopy2D(blobs_[0]->gpu_data(), w1, w, w1, w1, 1, cur_stream()));
      MC_CHECK(mcCopy2D(sibling_->blobs_[0]->gpu_data(), w2, w + w1, w2, w2, 1, cur_stream()));
      if (any_bias) {
        merged_bias_.Reshape(vector<int>{m1 + m2});
        float* b = merged_bias_.mutable_gpu_data();
        if (bias_term_) {
          MC_CHECK(mcCopy2D(blobs_[1]->gpu_data(), m1, b, m1, m1, 1, cur_stream()));
        } else {
          MC_CHECK(mcFill(b, m1, 0.f, cur_stream()));
        }
        if (sibling_->bias_term_) {
          MC_CHECK(mcCopy2D(sibling_->blobs_[1]->gpu_data(), m2, b + m1, m2, m2, 1, cur_stream()));
        } else {
          MC_CHECK(mcFill(b + m1, m2, 0.f, cur_stream()));
        }
      }
      MC_CHECK(mcConvPlanSetWeights(merged_plan_, merged_filter_.gpu_data(), cur_stream()));
      merged_version_ = v;
    }
    const int num = bottom[0]->shape(0);
    mcEpilogue ep = {nullptr, any_bias ? merged_bias_.gpu_data() : nullptr, nullptr, MC_ACT_NONE, 0.f};
    MC_CHECK(mcConvForwardTwoTops(merged_plan_, num, bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), m1,
                                  sibling_top_->mutable_gpu_data(), &ep, cur_stream()));
  }

  ConvolutionLayer* sibling_ = nullptr;
  Blob* sibling_top_ = nullptr;
  mcConvPlan* merged_plan_ = nullptr;
  int merged_h_ = -1, merged_w_in_ = -1, merged_m_ = -1;
  uint64_t merged_version_ = ~0ull;
  Blob merged_filter_, merged_bias_;
};
REGISTER_LAYER_CLASS(Convolution);

class DeconvolutionLayer : public BaseConvolutionLayer {
 public:
  explicit DeconvolutionLayer(const LayerParameter& param) : BaseConvolutionLayer(param) {}
  const char* type() const override { return "Deconvolution"; }

 protected:
  bool transposed() const override { return true; }
};
REGISTER_LAYER_CLASS(Deconvolution);

// ConvolutionDepthwise (reference src/layers/conv_dw_layer.cpp:9-158; .cu:9-72):
// reads convolution_param, filter blob [channels, 1, kernel_h, kernel_w], output
// channels = input channels.  Runs on the convolution plan's depthwise kernel.
class ConvolutionDepthwiseLayer : public BaseConvolutionLayer {
 public:
  explicit ConvolutionDepthwiseLayer(const LayerParameter& param) : BaseConvolutionLayer(param) {}
  const char* type() const override { return "ConvolutionDepthwise"; }

 protected:
  bool transposed() const override { return false; }
  bool depthwise() const override { return true; }
};
REGISTER_LAYER_CLASS(ConvolutionDepthwise);

// ---------------------------------------------------------------------------
// InnerProduct (reference src/layers/inner_product_layer.cpp:9-99; .cu:9-31)
// ---------------------------------------------------------------------------
class InnerProductLayer : public ContractionLayer {
 public:
  explicit InnerProductLayer(const LayerParameter& param) : ContractionLayer(param) {}
  const char* type() const override { return "InnerProduct"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("inner_product_param");
    N_ = static_cast<int>(p.get_int("num_output", 0));
    CHECK_GT(N_, 0);
    bias_term_ = p.get_bool("bias_term", true);
    transpose_ = p.get_bool("transpose", false);
    const int axis = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("axis", 1)));
    axis_ = axis;
    K_ = bottom[0]->count(axis);
    if (blobs_.empty()) {
      blobs_.resize(bias_term_ ? 2 : 1);
      blobs_[0].reset(new Blob(transpose_ ? vector<int>{K_, N_} : vector<int>{N_, K_}));
      FillConstant(p.sub("weight_filler"), blobs_[0].get());
      if (bias_term_) {
        blobs_[1].reset(new Blob(vector<int>{N_}));
        FillConstant(p.sub("bias_filler"), blobs_[1].get());
      }
    }
  }

  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("inner_product_param");
    const int axis = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("axis", 1)));
    CHECK_EQ(K_, bottom[0]->count(axis)) << "Input size incompatible with inner product parameters.";
    M_ = bottom[0]->count(0, axis);
    vector<int> top_shape = bottom[0]->shape();
    top_shape.resize(axis + 1);
    top_shape[axis] = N_;
    top[0]->Reshape(top_shape);
  }

  // Followers fold only when axis 1 of the top is the output unit.
  bool AcceptsEpilogue() const override { return axis_ == 1; }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (!plan_) MC_CHECK(mcInnerProductPlanCreate(K_, N_, transpose_ ? 1 : 0, &plan_));
    SyncWeights();
    mcEpilogue ep;
    PrepareEpilogue(N_, bias_term_ ? blobs_[1] : shared_ptr<Blob>(), &ep);
    if (M_ > 0)
      MC_CHECK(mcConvForward(plan_, M_, bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), &ep,
                             cur_stream()));
  }

  int M_ = 0, K_ = 0, N_ = 0, axis_ = 1;
  bool bias_term_ = true, transpose_ = false;
};
REGISTER_LAYER_CLASS(InnerProduct);

// ---------------------------------------------------------------------------
// BatchNorm (reference src/layers/batch_norm_layer.cpp:9-136; .cu:9-73)
// ---------------------------------------------------------------------------
class BatchNormLayer : public Layer {
 public:
  explicit BatchNormLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "BatchNorm"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("batch_norm_param");
    use_global_stats_ = p.has("use_global_stats") ? p.get_bool("use_global_stats") : true;
    channels_ = bottom[0]->num_axes() == 1 ? 1 : bottom[0]->shape(1);
    eps_ = static_cast<float>(p.get_float("eps", 1e-5));
    if (blobs_.empty()) {
      blobs_.resize(3);
      blobs_[0].reset(new Blob(vector<int>{channels_}));
      blobs_[1].reset(new Blob(vector<int>{channels_}));
      blobs_[2].reset(new Blob(vector<int>{1}));
      for (auto& b : blobs_) {
        real_t* d = b->mutable_cpu_data();
        for (int i = 0; i < b->count(); ++i) d[i] = 0;
      }
    } else {
      CHECK_EQ(blobs_.size(), 3u) << "BatchNorm takes 3 parameter blobs";
    }
  }

  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom[0]->num_axes() > 1) CHECK_EQ(bottom[0]->shape(1), channels_);
    top[0]->ReshapeLike(*bottom[0]);
    mean_.Reshape(vector<int>{channels_});
    stdev_.Reshape(vector<int>{channels_});
  }

  bool IsChannelStage(int channels) const override {
    return use_global_stats_ && channels == channels_;
  }
  // When it runs as its own pass, an in-place Scale/Bias and activation that
  // follow ride along in that pass (the WGAN generator's BatchNorm with batch
  // statistics -> Scale -> ReLU becomes statistics + one pass).
  bool AcceptsEpilogue() const override { return true; }
  int MaxAffineFollowers() const override { return 1; }
  // This pass owns the stage's subtract / divide fields (mean and deviation), so
  // only followers that fill the multiply / add fields or the activation fit:
  // another BatchNorm or a BN would lose its own subtraction.
  bool AcceptsFollower(const Layer* f) const override {
    const string ty = f->type();
    return ty == "Scale" || ty == "Bias" || ty == "ReLU" || ty == "TanH" || ty == "Sigmoid";
  }
  void SetEpilogue(const vector<Layer*>& followers) override { followers_ = followers; }
  uint64_t ChannelStageVersion() const override {
    return (BlobVersion(blobs_[0]) * 31 + BlobVersion(blobs_[1])) * 31 + BlobVersion(blobs_[2]);
  }
  void GetChannelStage(mcChannelOp* op) override {
    StoredStats();
    op->sub = mean_.gpu_data();
    op->div = stdev_.gpu_data();
  }

 protected:
  void StoredStats() {
    const uint64_t v = ChannelStageVersion();
    if (v == stats_version_) return;
    MC_CHECK(mcBatchNormStored(blobs_[0]->gpu_data(), blobs_[1]->gpu_data(), blobs_[2]->gpu_data(),
                               eps_, channels_, mean_.mutable_gpu_data(),
                               stdev_.mutable_gpu_data(), cur_stream()));
    stats_version_ = v;
  }

  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const int num = bottom[0]->shape(0);
    const int spatial = bottom[0]->count() / std::max(1, channels_ * num);
    if (bottom[0]->count() == 0) return;
    if (use_global_stats_) {
      StoredStats();
    } else {
      MC_CHECK(mcBatchNormBatchStats(bottom[0]->gpu_data(), num, channels_, spatial, eps_,
                                     mean_.mutable_gpu_data(), stdev_.mutable_gpu_data(),
                                     cur_stream()));
      stats_version_ = ~0ull;
    }
    mcChannelOp op = {nullptr, nullptr, nullptr, nullptr, MC_ACT_NONE, 0.f};
    for (Layer* f : followers_) f->GetChannelStage(&op);  // fills mul / add / activation
    op.sub = mean_.gpu_data();
    op.div = stdev_.gpu_data();
    MC_CHECK(mcChannelTransform(bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), num, channels_,
                                spatial, &op, cur_stream()));
  }

  vector<Layer*> followers_;
  bool use_global_stats_ = true;
  int channels_ = 0;
  float eps_ = 1e-5f;
  Blob mean_, stdev_;
  uint64_t stats_version_ = ~0ull;
};
REGISTER_LAYER_CLASS(BatchNorm);

// ---------------------------------------------------------------------------
// BN (reference src/layers/bn_layer.cpp:14-147; .cu:9-80): the frozen, fused form
// top = (x - blobs[2][c]) * blobs[3][c] * blobs[0][c] + blobs[1][c]; blobs[3]
// holds the multiplier itself (the reference never takes a root of it).
// ---------------------------------------------------------------------------
class BNLayer : public Layer {
 public:
  explicit BNLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "BN"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("bn_param");
    CHECK_GE(bottom[0]->num_axes(), 2) << "BN needs a channel axis";
    channels_ = bottom[0]->shape(1);
    if (blobs_.empty()) {
      blobs_.resize(4);
      for (auto& b : blobs_) b.reset(new Blob(vector<int>{1, channels_}));
      FillConstant(p.sub("slope_filler"), blobs_[0].get());
      FillConstant(p.sub("bias_filler"), blobs_[1].get());
      Message zero, one;
      one.set("value", "1");
      FillConstant(zero, blobs_[2].get());
      FillConstant(one, blobs_[3].get());
    } else {
      CHECK_EQ(blobs_.size(), 4u) << "BN takes 4 parameter blobs (slope, bias, mean, multiplier)";
      for (auto& b : blobs_) CHECK_EQ(b->count(), channels_) << "BN parameter size mismatch";
    }
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_EQ(bottom[0]->shape(1), channels_);
    top[0]->ReshapeLike(*bottom[0]);
    scale_.Reshape(vector<int>{channels_});
  }

  bool IsChannelStage(int channels) const override { return channels == channels_; }
  uint64_t ChannelStageVersion() const override {
    uint64_t v = 0;
    for (auto& b : blobs_) v = v * 31 + BlobVersion(b);
    return v;
  }
  void GetChannelStage(mcChannelOp* op) override {
    const uint64_t v = ChannelStageVersion();
    if (v != scale_version_) {
      const float* both[2] = {blobs_[3]->gpu_data(), blobs_[0]->gpu_data()};
      MC_CHECK(mcEltwise(MC_ELT_PROD, 2, both, nullptr, channels_, scale_.mutable_gpu_data(),
                         MC_ACT_NONE, 0.f, cur_stream()));
      scale_version_ = v;
    }
    op->sub = blobs_[2]->gpu_data();
    op->mul = scale_.gpu_data();
    op->add = blobs_[1]->gpu_data();
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom[0]->count() == 0) return;
    mcChannelOp op = {nullptr, nullptr, nullptr, nullptr, MC_ACT_NONE, 0.f};
    GetChannelStage(&op);
    const int num = bottom[0]->shape(0);
    MC_CHECK(mcChannelTransform(bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), num, channels_,
                                bottom[0]->count() / (num * channels_), &op, cur_stream()));
  }
  int channels_ = 0;
  Blob scale_;
  uint64_t scale_version_ = ~0ull;
};
REGISTER_LAYER_CLASS(BN);

// ---------------------------------------------------------------------------
// Scale and Bias (reference src/layers/scale_layer.cpp:10-119, .cu:9-47;
// bias_layer.cpp:9-89, .cu:9-30).  Scale's optional bias is applied in the same
// pass instead of through an embedded Bias layer.
// ---------------------------------------------------------------------------
class BroadcastLayer : public Layer {
 public:
  explicit BroadcastLayer(const LayerParameter& param) : Layer(param) {}
  int MinBottomBlobs() const override { return 1; }
  int MaxBottomBlobs() const override { return 2; }
  int ExactNumTopBlobs() const override { return 1; }

 protected:
  // Creates the learned operand for `bottom` given axis / num_axes.
  shared_ptr<Blob> MakeOperand(const Blob& bottom, int axis_param, int num_axes, const char* what) {
    const int axis = bottom.CanonicalAxisIndex(axis_param);
    CHECK_GE(num_axes, -1) << "num_axes must be non-negative, or -1 to extend to the end of bottom[0]";
    if (num_axes >= 0)
      CHECK_GE(bottom.num_axes(), axis + num_axes)
          << what << " blob's shape extends past bottom[0]'s shape when applied starting with "
          << "bottom[0] axis = " << axis;
    vector<int> shape(bottom.shape().begin() + axis, num_axes == -1
                                                         ? bottom.shape().end()
                                                         : bottom.shape().begin() + axis + num_axes);
    return shared_ptr<Blob>(new Blob(shape));
  }
  // outer / dim / inner of the broadcast of `operand` over `bottom`.
  void Extents(const Blob& bottom, const Blob& operand, int axis_param, const char* what) {
    axis_ = operand.num_axes() == 0 ? 0 : bottom.CanonicalAxisIndex(axis_param);
    CHECK_GE(bottom.num_axes(), axis_ + operand.num_axes())
        << what << " blob's shape extends past bottom[0]'s shape when applied starting with "
        << "bottom[0] axis = " << axis_;
    for (int i = 0; i < operand.num_axes(); ++i)
      CHECK_EQ(bottom.shape(axis_ + i), operand.shape(i))
          << "dimension mismatch between bottom[0]->shape(" << axis_ + i << ") and " << what
          << "->shape(" << i << ")";
    outer_ = bottom.count(0, axis_);
    dim_ = operand.count();
    inner_ = bottom.count(axis_ + operand.num_axes());
  }
  int axis_ = 0, outer_ = 0, dim_ = 0, inner_ = 0;
};

class ScaleLayer : public BroadcastLayer {
 public:
  explicit ScaleLayer(const LayerParameter& param) : BroadcastLayer(param) {}
  const char* type() const override { return "Scale"; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("scale_param");
    bias_term_ = p.get_bool("bias_term", false);
    const int axis = static_cast<int>(p.get_int("axis", 1));
    const int num_axes = static_cast<int>(p.get_int("num_axes", 1));
    if (bottom.size() == 1 && blobs_.empty()) {
      blobs_.push_back(MakeOperand(*bottom[0], axis, num_axes, "scale"));
      Message filler = p.sub("filler");
      if (!p.has("filler")) {
        filler.set("type", "constant");
        filler.set("value", "1");  // identity by default
      }
      FillConstant(filler, blobs_[0].get());
      if (bias_term_) {
        blobs_.push_back(MakeOperand(*bottom[0], axis, num_axes, "bias"));
        FillConstant(p.sub("bias_filler"), blobs_[1].get());
      }
    } else if (bottom.size() == 2 && bias_term_ && blobs_.empty()) {
      blobs_.push_back(MakeOperand(*bottom[0], axis, bottom[1]->num_axes(), "bias"));
      FillConstant(p.sub("bias_filler"), blobs_[0].get());
    }
  }

  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("scale_param");
    const Blob* scale = bottom.size() > 1 ? bottom[1] : blobs_[0].get();
    Extents(*bottom[0], *scale, static_cast<int>(p.get_int("axis", 1)), "scale");
    if (bottom[0] != top[0]) top[0]->ReshapeLike(*bottom[0]);
    if (bias_term_) CHECK_EQ(bias_blob()->count(), dim_) << "bias and scale extents differ";
  }

  bool IsChannelStage(int channels) const override {
    return blobs_.size() == static_cast<size_t>(bias_term_ ? 2 : 1) && axis_ == 1 && outer_ > 0 &&
           dim_ == channels && blobs_[0]->count() == channels;
  }
  uint64_t ChannelStageVersion() const override {
    return BlobVersion(blobs_[0]) * 31 + (bias_term_ ? BlobVersion(blobs_.back()) : 0);
  }
  void GetChannelStage(mcChannelOp* op) override {
    op->mul = blobs_[0]->gpu_data();
    if (bias_term_) op->add = blobs_[1]->gpu_data();
  }

 protected:
  Blob* bias_blob() { return blobs_.back().get(); }
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom[0]->count() == 0) return;
    const Blob* scale = bottom.size() > 1 ? bottom[1] : blobs_[0].get();
    mcChannelOp op = {nullptr, nullptr, scale->gpu_data(),
                      bias_term_ ? bias_blob()->gpu_data() : nullptr, MC_ACT_NONE, 0.f};
    MC_CHECK(mcChannelTransform(bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), outer_, dim_,
                                inner_, &op, cur_stream()));
  }
  bool bias_term_ = false;
};
REGISTER_LAYER_CLASS(Scale);

class BiasLayer : public BroadcastLayer {
 public:
  explicit BiasLayer(const LayerParameter& param) : BroadcastLayer(param) {}
  const char* type() const override { return "Bias"; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("bias_param");
    if (bottom.size() == 1 && blobs_.empty()) {
      blobs_.push_back(MakeOperand(*bottom[0], static_cast<int>(p.get_int("axis", 1)),
                                   static_cast<int>(p.get_int("num_axes", 1)), "bias"));
      FillConstant(p.sub("filler"), blobs_[0].get());
    }
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("bias_param");
    const Blob* bias = bottom.size() > 1 ? bottom[1] : blobs_[0].get();
    Extents(*bottom[0], *bias, static_cast<int>(p.get_int("axis", 1)), "bias");
    if (bottom[0] != top[0]) top[0]->ReshapeLike(*bottom[0]);
  }
  bool IsChannelStage(int channels) const override {
    return blobs_.size() == 1 && axis_ == 1 && dim_ == channels;
  }
  uint64_t ChannelStageVersion() const override { return BlobVersion(blobs_[0]); }
  void GetChannelStage(mcChannelOp* op) override { op->add = blobs_[0]->gpu_data(); }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom[0]->count() == 0) return;
    const Blob* bias = bottom.size() > 1 ? bottom[1] : blobs_[0].get();
    mcChannelOp op = {nullptr, nullptr, nullptr, bias->gpu_data(), MC_ACT_NONE, 0.f};
    MC_CHECK(mcChannelTransform(bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), outer_, dim_,
                                inner_, &op, cur_stream()));
  }
};
REGISTER_LAYER_CLASS(Bias);

// ---------------------------------------------------------------------------
// ReLU / TanH / Sigmoid (reference relu_layer.cpp:12-30, tanh_layer.cpp:14-22,
// sigmoid_layer.cpp:12-24; .cu twins)
// ---------------------------------------------------------------------------
class NeuronLayer : public Layer {
 public:
  explicit NeuronLayer(const LayerParameter& param) : Layer(param) {}
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    top[0]->ReshapeLike(*bottom[0]);
  }
  bool IsChannelStage(int) const override { return true; }
  void GetChannelStage(mcChannelOp* op) override {
    op->activation = activation();
    op->negative_slope = slope();
  }

 protected:
  virtual int activation() const = 0;
  virtual float slope() const { return 0.f; }
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom[0]->count() == 0) return;
    mcChannelOp op = {nullptr, nullptr, nullptr, nullptr, activation(), slope()};
    MC_CHECK(mcChannelTransform(bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), 1, 1,
                                bottom[0]->count(), &op, cur_stream()));
  }
};

class ReLULayer : public NeuronLayer {
 public:
  explicit ReLULayer(const LayerParameter& param) : NeuronLayer(param) {
    const float s = static_cast<float>(layer_param_.sub("relu_param").get_float("negative_slope", 0.));
    slope_ = std::abs(s) < 1e-6 ? 0.f : s;  // the CPU reference treats a tiny slope as none
  }
  const char* type() const override { return "ReLU"; }

 protected:
  int activation() const override { return MC_ACT_RELU; }
  float slope() const override { return slope_; }
  float slope_;
};
REGISTER_LAYER_CLASS(ReLU);

class TanHLayer : public NeuronLayer {
 public:
  explicit TanHLayer(const LayerParameter& param) : NeuronLayer(param) {}
  const char* type() const override { return "TanH"; }

 protected:
  int activation() const override { return MC_ACT_TANH; }
};
REGISTER_LAYER_CLASS(TanH);

class SigmoidLayer : public NeuronLayer {
 public:
  explicit SigmoidLayer(const LayerParameter& param) : NeuronLayer(param) {}
  const char* type() const override { return "Sigmoid"; }

 protected:
  int activation() const override { return MC_ACT_SIGMOID; }
};
REGISTER_LAYER_CLASS(Sigmoid);

// ---------------------------------------------------------------------------
// Pooling (reference src/layers/pooling_layer.cpp:17-189; .cu:10-99)
// ---------------------------------------------------------------------------
class PoolingLayer : public Layer {
 public:
  explicit PoolingLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Pooling"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("pooling_param");
    global_ = p.get_bool("global_pooling", false);
    if (global_) {
      CHECK(!(p.has("kernel_size") || p.has("kernel_h") || p.has("kernel_w")))
          << "With Global_pooling: true Filter size cannot specified";
    } else {
      CHECK(!p.has("kernel_size") != !(p.has("kernel_h") && p.has("kernel_w")))
          << "Filter size is kernel_size OR kernel_h and kernel_w; not both";
      CHECK(p.has("kernel_size") || (p.has("kernel_h") && p.has("kernel_w")))
          << "For non-square filters both kernel_h and kernel_w are required.";
    }
    CHECK((!p.has("pad") && p.has("pad_h") && p.has("pad_w")) || (!p.has("pad_h") && !p.has("pad_w")))
        << "pad is pad OR pad_h and pad_w are required.";
    CHECK((!p.has("stride") && p.has("stride_h") && p.has("stride_w")) ||
          (!p.has("stride_h") && !p.has("stride_w")))
        << "Stride is stride OR stride_h and stride_w are required.";
    const string method = p.get_string("pool", "MAX");
    if (method == "MAX" || method == "0") method_ = MC_POOL_MAX;
    else if (method == "AVE" || method == "1") method_ = MC_POOL_AVE;
    else LOG(FATAL) << "Unknown pooling method.";
    if (global_) {
      kh_ = bottom[0]->height();
      kw_ = bottom[0]->width();
    } else if (p.has("kernel_size")) {
      kh_ = kw_ = static_cast<int>(p.get_int("kernel_size"));
    } else {
      kh_ = static_cast<int>(p.get_int("kernel_h"));
      kw_ = static_cast<int>(p.get_int("kernel_w"));
    }
    CHECK_GT(kh_, 0) << "Filter dimensions cannot be zero.";
    CHECK_GT(kw_, 0) << "Filter dimensions cannot be zero.";
    if (!p.has("pad_h")) ph_ = pw_ = static_cast<int>(p.get_int("pad", 0));
    else {
      ph_ = static_cast<int>(p.get_int("pad_h"));
      pw_ = static_cast<int>(p.get_int("pad_w"));
    }
    if (!p.has("stride_h")) sh_ = sw_ = static_cast<int>(p.get_int("stride", 1));
    else {
      sh_ = static_cast<int>(p.get_int("stride_h"));
      sw_ = static_cast<int>(p.get_int("stride_w"));
    }
    if (global_)
      CHECK(ph_ == 0 && pw_ == 0 && sh_ == 1 && sw_ == 1)
          << "With Global_pooling: true; only pad = 0 and stride = 1";
    if (ph_ != 0 || pw_ != 0) {
      CHECK_LT(ph_, kh_);
      CHECK_LT(pw_, kw_);
    }
  }

  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_EQ(4, bottom[0]->num_axes()) << "Input must have 4 axes, corresponding to "
                                       << "(num, channels, height, width)";
    if (global_) {
      kh_ = bottom[0]->height();
      kw_ = bottom[0]->width();
    }
    int ho, wo;
    MC_CHECK(mcPoolingOutputShape(bottom[0]->height(), bottom[0]->width(), kh_, kw_, sh_, sw_, ph_,
                                  pw_, &ho, &wo));
    top[0]->Reshape(bottom[0]->num(), bottom[0]->channels(), ho, wo);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    MC_CHECK(mcPooling(method_, bottom[0]->gpu_data(), top[0]->mutable_gpu_data(),
                       bottom[0]->num() * bottom[0]->channels(), bottom[0]->height(),
                       bottom[0]->width(), kh_, kw_, sh_, sw_, ph_, pw_, cur_stream()));
  }
  int method_ = MC_POOL_MAX;
  bool global_ = false;
  int kh_ = 0, kw_ = 0, sh_ = 1, sw_ = 1, ph_ = 0, pw_ = 0;
};
REGISTER_LAYER_CLASS(Pooling);

// ---------------------------------------------------------------------------
// Eltwise (reference src/layers/eltwise_layer.cpp:9-78; .cu:10-50).  An in-place
// activation that directly follows is applied in the same pass.
// ---------------------------------------------------------------------------
class EltwiseLayer : public Layer {
 public:
  explicit EltwiseLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Eltwise"; }
  int MinBottomBlobs() const override { return 2; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("eltwise_param");
    const int nc = p.count("coeff");
    CHECK(nc == 0 || nc == static_cast<int>(bottom.size()))
        << "Eltwise Layer takes one coefficient per bottom blob.";
    const string op = p.get_string("operation", "SUM");
    if (op == "PROD" || op == "0") op_ = MC_ELT_PROD;
    else if (op == "SUM" || op == "1") op_ = MC_ELT_SUM;
    else if (op == "MAX" || op == "2") op_ = MC_ELT_MAX;
    else LOG(FATAL) << "Unknown elementwise operation.";
    CHECK(!(op_ == MC_ELT_PROD && nc)) << "Eltwise layer only takes coefficients for summation.";
    CHECK_LE(bottom.size(), 8u) << "Eltwise: at most 8 bottoms are supported";
    coeffs_.assign(bottom.size(), 1.f);
    for (int i = 0; i < nc; ++i) coeffs_[i] = static_cast<float>(p.get_float("coeff", 1., i));
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    for (size_t i = 1; i < bottom.size(); ++i) CHECK(bottom[i]->shape() == bottom[0]->shape());
    top[0]->ReshapeLike(*bottom[0]);
  }
  bool AcceptsEpilogue() const override { return true; }
  void SetEpilogue(const vector<Layer*>& followers) override {
    // Only a lone activation can ride along.
    act_follower_ = nullptr;
    CHECK(followers.size() <= 1) << "Eltwise can absorb a single activation";
    if (!followers.empty()) act_follower_ = followers[0];
  }
  bool IsPlainSum() const override {
    return op_ == MC_ELT_SUM && coeffs_.size() == 2 && coeffs_[0] == 1.f && coeffs_[1] == 1.f;
  }
  Layer* AbsorbedActivation() const override { return act_follower_; }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const float* ptrs[8];
    for (size_t i = 0; i < bottom.size(); ++i) ptrs[i] = bottom[i]->gpu_data();
    mcChannelOp act = {nullptr, nullptr, nullptr, nullptr, MC_ACT_NONE, 0.f};
    if (act_follower_) act_follower_->GetChannelStage(&act);
    MC_CHECK(mcEltwise(op_, static_cast<int>(bottom.size()), ptrs, coeffs_.data(),
                       top[0]->count(), top[0]->mutable_gpu_data(), act.activation,
                       act.negative_slope, cur_stream()));
  }
  int op_ = MC_ELT_SUM;
  vector<float> coeffs_;
  Layer* act_follower_ = nullptr;
};
REGISTER_LAYER_CLASS(Eltwise);

// ---------------------------------------------------------------------------
// Softmax (reference src/layers/softmax_layer.cpp:13-63; .cu:77-111)
// ---------------------------------------------------------------------------
class SoftmaxLayer : public Layer {
 public:
  explicit SoftmaxLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Softmax"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    axis_ = bottom[0]->CanonicalAxisIndex(
        static_cast<int>(layer_param_.sub("softmax_param").get_int("axis", 1)));
    top[0]->ReshapeLike(*bottom[0]);
    outer_ = bottom[0]->count(0, axis_);
    inner_ = bottom[0]->count(axis_ + 1);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom[0]->count() == 0) return;
    const float* x = bottom[0]->gpu_data();
    float* y = top[0]->mutable_gpu_data();
    if (x == y && inner_ != 1) {
      // the column kernel cannot run in place: stage through a scratch blob
      scratch_.ReshapeLike(*bottom[0]);
      MC_CHECK(mcCopy2D(x, bottom[0]->count(), scratch_.mutable_gpu_data(), bottom[0]->count(),
                        bottom[0]->count(), 1, cur_stream()));
      x = scratch_.gpu_data();
    }
    MC_CHECK(mcSoftmax(x, y, outer_, bottom[0]->shape(axis_), inner_, cur_stream()));
  }
  int axis_ = 1, outer_ = 0, inner_ = 0;
  Blob scratch_;
};
REGISTER_LAYER_CLASS(Softmax);

}  // namespace caffe
