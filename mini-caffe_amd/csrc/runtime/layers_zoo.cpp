// The less common layers of the model zoo: Dropout, Power, Exp, Log, AbsVal, BNLL,
// ELU, Threshold, PReLU, LRN, ArgMax, Reduction, MVN, Embed, Filter, Crop, Tile,
// ShuffleChannel, SPP, Parameter.
//
// Host-side set-up and shape inference restate the reference layer of the same
// name (file:line given per class); Forward_gpu hands device pointers to the
// kernel ABI in mchip/kernels.h on the calling thread's stream.
#include <algorithm>
#include <cmath>

#include "layer.hpp"

namespace caffe {

namespace {

// One bottom, one top of the same shape (reference src/layers/neuron_layer.cpp:7-10).
class SameShapeLayer : public Layer {
 public:
  explicit SameShapeLayer(const LayerParameter& param) : Layer(param) {}
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    top[0]->ReshapeLike(*bottom[0]);
  }
};

// A SameShapeLayer that is one mcUnary call.
class UnaryLayer : public SameShapeLayer {
 public:
  explicit UnaryLayer(const LayerParameter& param) : SameShapeLayer(param) {}

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    MC_CHECK(mcUnary(op_, bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), bottom[0]->count(),
                     p0_, p1_, p2_, cur_stream()));
  }
  int op_ = MC_UNARY_ABS;
  float p0_ = 0.f, p1_ = 0.f, p2_ = 0.f;
};

}  // namespace

// ---------------------------------------------------------------------------
// Dropout (reference src/layers/dropout_layer.cpp:8-16; .cu:7-14): inference
// only, a copy; nothing to do when it runs in place.
// ---------------------------------------------------------------------------
class DropoutLayer : public SameShapeLayer {
 public:
  explicit DropoutLayer(const LayerParameter& param) : SameShapeLayer(param) {}
  const char* type() const override { return "Dropout"; }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom[0] != top[0]) DeviceCopy(*bottom[0], top[0]);
  }
};
REGISTER_LAYER_CLASS(Dropout);

// ---------------------------------------------------------------------------
// Power (reference src/layers/power_layer.cpp:8-40; .cu:8-29): (shift + scale*x)^power
// ---------------------------------------------------------------------------
class PowerLayer : public UnaryLayer {
 public:
  explicit PowerLayer(const LayerParameter& param) : UnaryLayer(param) {
    const Message& p = layer_param_.sub("power_param");
    op_ = MC_UNARY_POWER;
    p0_ = static_cast<float>(p.get_float("scale", 1.));
    p1_ = static_cast<float>(p.get_float("shift", 0.));
    p2_ = static_cast<float>(p.get_float("power", 1.));
  }
  const char* type() const override { return "Power"; }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (p2_ * p0_ == 0.f) {
      // The input does not matter: scale or power is 0.
      const float value = p2_ == 0.f ? 1.f : std::pow(p1_, p2_);
      MC_CHECK(mcFill(top[0]->mutable_gpu_data(), top[0]->count(), value, cur_stream()));
      return;
    }
    UnaryLayer::Forward_gpu(bottom, top);
  }
};
REGISTER_LAYER_CLASS(Power);

// ---------------------------------------------------------------------------
// Exp (reference src/layers/exp_layer.cpp:8-45): base^(shift + scale*x), computed
// as base^shift * exp(log(base)*scale * x); base -1 means e.
// ---------------------------------------------------------------------------
class ExpLayer : public UnaryLayer {
 public:
  explicit ExpLayer(const LayerParameter& param) : UnaryLayer(param) {
    const Message& p = layer_param_.sub("exp_param");
    const float base = static_cast<float>(p.get_float("base", -1.));
    if (base != -1.f) CHECK_GT(base, 0) << "base must be strictly positive.";
    const float log_base = base == -1.f ? 1.f : std::log(base);
    CHECK(!std::isnan(log_base)) << "NaN result: log(base) = log(" << base << ") = " << log_base;
    CHECK(!std::isinf(log_base)) << "Inf result: log(base) = log(" << base << ") = " << log_base;
    const float scale = static_cast<float>(p.get_float("scale", 1.));
    const float shift = static_cast<float>(p.get_float("shift", 0.));
    op_ = MC_UNARY_EXP;
    p0_ = log_base * scale;
    p1_ = shift == 0.f ? 1.f : (base != -1.f ? std::pow(base, shift) : std::exp(shift));
  }
  const char* type() const override { return "Exp"; }
};
REGISTER_LAYER_CLASS(Exp);

// ---------------------------------------------------------------------------
// Log (reference src/layers/log_layer.cpp:8-54): log_base(shift + scale*x)
// ---------------------------------------------------------------------------
class LogLayer : public UnaryLayer {
 public:
  explicit LogLayer(const LayerParameter& param) : UnaryLayer(param) {
    const Message& p = layer_param_.sub("log_param");
    const float base = static_cast<float>(p.get_float("base", -1.));
    if (base != -1.f) CHECK_GT(base, 0) << "base must be strictly positive.";
    const float log_base = base == -1.f ? 1.f : std::log(base);
    CHECK(!std::isnan(log_base)) << "NaN result: log(base) = log(" << base << ") = " << log_base;
    CHECK(!std::isinf(log_base)) << "Inf result: log(base) = log(" << base << ") = " << log_base;
    const float base_scale = 1.f / log_base;
    CHECK(!std::isnan(base_scale))
        << "NaN result: 1/log(base) = 1/log(" << base << ") = " << base_scale;
    CHECK(!std::isinf(base_scale))
        << "Inf result: 1/log(base) = 1/log(" << base << ") = " << base_scale;
    op_ = MC_UNARY_LOG;
    p0_ = static_cast<float>(p.get_float("scale", 1.));
    p1_ = static_cast<float>(p.get_float("shift", 0.));
    p2_ = base_scale;
  }
  const char* type() const override { return "Log"; }
};
REGISTER_LAYER_CLASS(Log);

// ---------------------------------------------------------------------------
// AbsVal, BNLL, ELU, Threshold (reference absval_layer.cpp:8-13,
// bnll_layer.cpp:8-18, elu_layer.cpp:8-18, threshold_layer.cpp:7-21)
// ---------------------------------------------------------------------------
class AbsValLayer : public UnaryLayer {
 public:
  explicit AbsValLayer(const LayerParameter& param) : UnaryLayer(param) { op_ = MC_UNARY_ABS; }
  const char* type() const override { return "AbsVal"; }
};
REGISTER_LAYER_CLASS(AbsVal);

class BNLLLayer : public UnaryLayer {
 public:
  explicit BNLLLayer(const LayerParameter& param) : UnaryLayer(param) { op_ = MC_UNARY_BNLL; }
  const char* type() const override { return "BNLL"; }
};
REGISTER_LAYER_CLASS(BNLL);

class ELULayer : public UnaryLayer {
 public:
  explicit ELULayer(const LayerParameter& param) : UnaryLayer(param) {
    op_ = MC_UNARY_ELU;
    p0_ = static_cast<float>(layer_param_.sub("elu_param").get_float("alpha", 1.));
  }
  const char* type() const override { return "ELU"; }
};
REGISTER_LAYER_CLASS(ELU);

class ThresholdLayer : public UnaryLayer {
 public:
  explicit ThresholdLayer(const LayerParameter& param) : UnaryLayer(param) {
    op_ = MC_UNARY_THRESHOLD;
    p0_ = static_cast<float>(layer_param_.sub("threshold_param").get_float("threshold", 0.));
  }
  const char* type() const override { return "Threshold"; }
};
REGISTER_LAYER_CLASS(Threshold);

// ---------------------------------------------------------------------------
// PReLU (reference src/layers/prelu_layer.cpp:9-84; .cu:9-33)
// ---------------------------------------------------------------------------
class PReLULayer : public SameShapeLayer {
 public:
  explicit PReLULayer(const LayerParameter& param) : SameShapeLayer(param) {}
  const char* type() const override { return "PReLU"; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_GE(bottom[0]->num_axes(), 2) << "Number of axes of bottom blob must be >=2.";
    const Message& p = layer_param_.sub("prelu_param");
    const int channels = bottom[0]->shape(1);
    channel_shared_ = p.get_bool("channel_shared", false);
    if (blobs_.empty()) {
      blobs_.resize(1);
      blobs_[0].reset(new Blob(channel_shared_ ? vector<int>() : vector<int>(1, channels)));
      FillConstant(p.sub("filler"), blobs_[0].get(), p.has("filler") ? 0. : 0.25);
    }
    CHECK_EQ(blobs_[0]->count(), channel_shared_ ? 1 : channels)
        << "Negative slope size is inconsistent with prototxt config";
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_GE(bottom[0]->num_axes(), 2) << "Number of axes of bottom blob must be >=2.";
    top[0]->ReshapeLike(*bottom[0]);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom[0]->count() == 0) return;
    MC_CHECK(mcPReLU(bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), bottom[0]->shape(0),
                     bottom[0]->shape(1), bottom[0]->count(2), blobs_[0]->gpu_data(),
                     channel_shared_ ? 1 : 0, cur_stream()));
  }
  bool channel_shared_ = false;
};
REGISTER_LAYER_CLASS(PReLU);

// ---------------------------------------------------------------------------
// LRN (reference src/layers/lrn_layer.cpp:13-164; .cu:9-94).  The within-channel
// region, a chain of five layers there, is one kernel here.
// ---------------------------------------------------------------------------
class LRNLayer : public Layer {
 public:
  explicit LRNLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "LRN"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("lrn_param");
    size_ = static_cast<int>(p.get_int("local_size", 5));
    CHECK_EQ(size_ % 2, 1) << "LRN only supports odd values for local_size";
    alpha_ = static_cast<float>(p.get_float("alpha", 1.));
    beta_ = static_cast<float>(p.get_float("beta", 0.75));
    k_ = static_cast<float>(p.get_float("k", 1.));
    const string region = p.get_string("norm_region", "ACROSS_CHANNELS");
    if (region == "ACROSS_CHANNELS" || region == "0") {
      within_ = false;
    } else if (region == "WITHIN_CHANNEL" || region == "1") {
      within_ = true;
    } else {
      LOG(FATAL) << "Unknown normalization region.";
    }
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_EQ(4, bottom[0]->num_axes())
        << "Input must have 4 axes, corresponding to (num, channels, height, width)";
    CHECK(bottom[0] != top[0]) << "LRN cannot run in place";
    top[0]->ReshapeLike(*bottom[0]);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Blob& b = *bottom[0];
    if (b.count() == 0) return;
    if (within_) {
      MC_CHECK(mcLRNWithinChannel(b.gpu_data(), top[0]->mutable_gpu_data(),
                                  static_cast<long>(b.shape(0)) * b.shape(1), b.shape(2),
                                  b.shape(3), size_, alpha_, beta_, cur_stream()));
    } else {
      MC_CHECK(mcLRNAcrossChannels(b.gpu_data(), top[0]->mutable_gpu_data(), b.shape(0),
                                   b.shape(1), b.shape(2), b.shape(3), size_, alpha_, beta_, k_,
                                   cur_stream()));
    }
  }
  int size_ = 5;
  float alpha_ = 1.f, beta_ = 0.75f, k_ = 1.f;
  bool within_ = false;
};
REGISTER_LAYER_CLASS(LRN);

// ---------------------------------------------------------------------------
// ArgMax (reference src/layers/argmax_layer.cpp:11-93; host code only there)
// ---------------------------------------------------------------------------
class ArgMaxLayer : public Layer {
 public:
  explicit ArgMaxLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "ArgMax"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("argmax_param");
    out_max_val_ = p.get_bool("out_max_val", false);
    top_k_ = static_cast<int>(p.get_int("top_k", 1));
    has_axis_ = p.has("axis");
    CHECK_GE(top_k_, 1) << "top k must not be less than 1.";
    if (has_axis_) {
      axis_ = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("axis", 0)));
      CHECK_LE(top_k_, bottom[0]->shape(axis_))
          << "top_k must be less than or equal to the dimension of the axis.";
    } else {
      CHECK_LE(top_k_, bottom[0]->count(1))
          << "top_k must be less than or equal to the dimension of the flattened bottom blob "
             "per instance.";
    }
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK(bottom[0] != top[0]) << "ArgMax cannot run in place";
    vector<int> shape(std::max(3, bottom[0]->num_axes()), 1);
    if (has_axis_) {
      shape = bottom[0]->shape();
      shape[axis_] = top_k_;
    } else {
      shape[0] = bottom[0]->shape(0);
      shape[2] = top_k_;
      if (out_max_val_) shape[1] = 2;
    }
    top[0]->Reshape(shape);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Blob& b = *bottom[0];
    if (b.count() == 0) return;
    const int dim = has_axis_ ? b.shape(axis_) : b.count(1);
    const int inner = has_axis_ ? b.count(axis_ + 1) : 1;
    const long outer = has_axis_ ? b.count(0, axis_) : b.shape(0);
    const int layout = !out_max_val_ ? MC_ARGMAX_INDEX
                                     : (has_axis_ ? MC_ARGMAX_VALUE : MC_ARGMAX_INDEX_THEN_VALUE);
    MC_CHECK(mcArgMax(b.gpu_data(), top[0]->mutable_gpu_data(), outer, dim, inner, top_k_, layout,
                      cur_stream()));
  }
  bool out_max_val_ = false, has_axis_ = false;
  int top_k_ = 1, axis_ = 0;
};
REGISTER_LAYER_CLASS(ArgMax);

// ---------------------------------------------------------------------------
// Reduction (reference src/layers/reduction_layer.cpp:8-72; .cu:8-40)
// ---------------------------------------------------------------------------
class ReductionLayer : public Layer {
 public:
  explicit ReductionLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Reduction"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const string op = layer_param_.sub("reduction_param").get_string("operation", "SUM");
    if (op == "SUM" || op == "1") {
      op_ = MC_REDUCE_SUM;
    } else if (op == "ASUM" || op == "2") {
      op_ = MC_REDUCE_ASUM;
    } else if (op == "SUMSQ" || op == "3") {
      op_ = MC_REDUCE_SUMSQ;
    } else if (op == "MEAN" || op == "4") {
      op_ = MC_REDUCE_MEAN;
    } else {
      LOG(FATAL) << "Unknown reduction op: " << op;
    }
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("reduction_param");
    CHECK(bottom[0] != top[0]) << "Reduction cannot run in place";
    const int axis = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("axis", 0)));
    num_ = bottom[0]->count(0, axis);
    dim_ = bottom[0]->count(axis);
    top[0]->Reshape(
        vector<int>(bottom[0]->shape().begin(), bottom[0]->shape().begin() + axis));
    CHECK_EQ(num_, top[0]->count());
    coeff_ = static_cast<float>(p.get_float("coeff", 1.));
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (num_ == 0 || dim_ == 0) return;
    MC_CHECK(mcReduction(op_, bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), num_, dim_,
                         coeff_, cur_stream()));
  }
  int op_ = MC_REDUCE_SUM, num_ = 0, dim_ = 0;
  float coeff_ = 1.f;
};
REGISTER_LAYER_CLASS(Reduction);

// ---------------------------------------------------------------------------
// MVN (reference src/layers/mvn_layer.cpp:8-75; .cu:8-49)
// ---------------------------------------------------------------------------
class MVNLayer : public Layer {
 public:
  explicit MVNLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "MVN"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("mvn_param");
    CHECK_LE(bottom[0]->num_axes(), 4) << "MVN takes blobs of at most 4 axes";
    // The reference reshapes through the legacy 4-D accessors: missing axes are 1.
    vector<int> shape(4, 1);
    for (int i = 0; i < bottom[0]->num_axes(); ++i) shape[i] = bottom[0]->shape(i);
    if (bottom[0] != top[0]) top[0]->Reshape(shape);
    across_channels_ = p.get_bool("across_channels", false);
    normalize_variance_ = p.get_bool("normalize_variance", true);
    eps_ = static_cast<float>(p.get_float("eps", 1e-9));
    num_ = across_channels_ ? shape[0] : shape[0] * shape[1];
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom[0]->count() == 0) return;
    MC_CHECK(mcMVN(bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), num_,
                   bottom[0]->count() / num_, normalize_variance_ ? 1 : 0, eps_, cur_stream()));
  }
  bool across_channels_ = false, normalize_variance_ = true;
  float eps_ = 1e-9f;
  int num_ = 0;
};
REGISTER_LAYER_CLASS(MVN);

// ---------------------------------------------------------------------------
// Embed (reference src/layers/embed_layer.cpp:9-79; .cu:9-35)
// ---------------------------------------------------------------------------
class EmbedLayer : public Layer {
 public:
  explicit EmbedLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Embed"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("embed_param");
    N_ = static_cast<int>(p.get_int("num_output", 0));
    CHECK_GT(N_, 0) << "EmbedLayer num_output must be positive.";
    K_ = static_cast<int>(p.get_int("input_dim", 0));
    CHECK_GT(K_, 0) << "EmbedLayer input_dim must be positive.";
    bias_term_ = p.get_bool("bias_term", true);
    if (blobs_.empty()) {
      blobs_.resize(bias_term_ ? 2 : 1);
      blobs_[0].reset(new Blob(vector<int>{K_, N_}));
      FillConstant(p.sub("weight_filler"), blobs_[0].get());
      if (bias_term_) {
        blobs_[1].reset(new Blob(vector<int>{N_}));
        FillConstant(p.sub("bias_filler"), blobs_[1].get());
      }
    } else {
      CHECK_EQ(blobs_.size(), static_cast<size_t>(bias_term_ ? 2 : 1));
      CHECK_EQ(blobs_[0]->count(), K_ * N_) << "Embed weight size mismatch";
    }
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK(bottom[0] != top[0]) << "Embed cannot run in place";
    vector<int> top_shape = bottom[0]->shape();
    top_shape.push_back(N_);
    top[0]->Reshape(top_shape);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    MC_CHECK(mcGatherRows(blobs_[0]->gpu_data(), K_, N_, bottom[0]->gpu_data(),
                          bottom[0]->count(), bias_term_ ? blobs_[1]->gpu_data() : nullptr,
                          top[0]->mutable_gpu_data(), cur_stream()));
  }
  int N_ = 0, K_ = 0;
  bool bias_term_ = true;
};
REGISTER_LAYER_CLASS(Embed);

// ---------------------------------------------------------------------------
// Filter (reference src/layers/filter_layer.cpp:8-75; .cu:7-23).  As there, the
// selector is read when the layer is reshaped, not when it runs.
// ---------------------------------------------------------------------------
class FilterLayer : public Layer {
 public:
  explicit FilterLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Filter"; }
  int MinBottomBlobs() const override { return 2; }
  int MinTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_EQ(top.size(), bottom.size() - 1);
    first_reshape_ = true;
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Blob& selector = *bottom.back();
    for (int i = 1; i < selector.num_axes(); ++i)
      CHECK_EQ(selector.shape(i), 1)
          << "Selector blob dimensions must be singletons (1), except the first";
    for (size_t i = 0; i + 1 < bottom.size(); ++i) {
      CHECK_EQ(selector.shape(0), bottom[i]->shape(0))
          << "Each bottom should have the same 0th dimension as the selector blob";
      CHECK(bottom[i] != top[i]) << "Filter cannot run in place";
    }
    const real_t* sel = selector.cpu_data();
    vector<float> rows;
    for (int item = 0; item < selector.shape(0); ++item)
      if (sel[item]) rows.push_back(static_cast<float>(item));
    kept_ = static_cast<int>(rows.size());
    rows_.Reshape(vector<int>{std::max(kept_, 1)});
    std::copy(rows.begin(), rows.end(), rows_.mutable_cpu_data());
    int new_tops_num = kept_;
    if (first_reshape_) {
      new_tops_num = bottom[0]->shape(0);
      first_reshape_ = false;
    }
    for (size_t t = 0; t < top.size(); ++t) {
      vector<int> shape = bottom[t]->shape();
      shape[0] = new_tops_num;
      top[t]->Reshape(shape);
    }
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (kept_ == 0) return;
    for (size_t t = 0; t < top.size(); ++t) {
      const int dim = bottom[t]->count(1);
      if (dim == 0) continue;
      MC_CHECK(mcGatherRows(bottom[t]->gpu_data(), bottom[t]->shape(0), dim, rows_.gpu_data(),
                            kept_, nullptr, top[t]->mutable_gpu_data(), cur_stream()));
    }
  }
  bool first_reshape_ = true;
  int kept_ = 0;
  Blob rows_;  // kept item numbers, as floats
};
REGISTER_LAYER_CLASS(Filter);

// ---------------------------------------------------------------------------
// Crop (reference src/layers/crop_layer.cpp:12-107; .cu:11-80)
// ---------------------------------------------------------------------------
class CropLayer : public Layer {
 public:
  explicit CropLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Crop"; }
  int ExactNumBottomBlobs() const override { return 2; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("crop_param");
    CHECK_EQ(bottom.size(), 2u) << "Wrong number of bottom blobs.";
    const int input_dim = bottom[0]->num_axes();
    const int start_axis = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("axis", 2)));
    CHECK_LT(start_axis, input_dim) << "crop axis bigger than input dim";
    if (p.count("offset") > 1)
      CHECK_EQ(start_axis + p.count("offset"), input_dim)
          << "number of offset values specified must be equal to the number of "
          << "dimensions following axis.";
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("crop_param");
    CHECK(bottom[0] != top[0]) << "Crop cannot run in place";
    const int input_dim = bottom[0]->num_axes();
    CHECK_LE(input_dim, MC_MAX_AXES) << "Crop takes blobs of at most " << MC_MAX_AXES << " axes";
    const int start_axis = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("axis", 2)));
    const int n_off = p.count("offset");
    offsets_.assign(input_dim, 0);
    vector<int> new_shape(bottom[0]->shape());
    for (int i = start_axis; i < input_dim; ++i) {
      int crop_offset = 0;
      if (n_off == 1) {
        crop_offset = static_cast<int>(p.get_int("offset", 0, 0));
      } else if (n_off > 1) {
        crop_offset = static_cast<int>(p.get_int("offset", 0, i - start_axis));
      }
      CHECK_GE(bottom[0]->shape(i) - crop_offset, bottom[1]->shape(i))
          << "the crop for dimension " << i << " is out-of-bounds with size "
          << bottom[1]->shape(i) << " and offset " << crop_offset;
      new_shape[i] = bottom[1]->shape(i);
      offsets_[i] = crop_offset;
    }
    top[0]->Reshape(new_shape);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (top[0]->count() == 0) return;
    MC_CHECK(mcCrop(bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), bottom[0]->num_axes(),
                    bottom[0]->shape().data(), top[0]->shape().data(), offsets_.data(),
                    cur_stream()));
  }
  vector<int> offsets_;
};
REGISTER_LAYER_CLASS(Crop);

// ---------------------------------------------------------------------------
// Tile (reference src/layers/tile_layer.cpp:8-35; .cu:9-29)
// ---------------------------------------------------------------------------
class TileLayer : public Layer {
 public:
  explicit TileLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Tile"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("tile_param");
    CHECK(bottom[0] != top[0]) << "Tile cannot run in place";
    const int axis = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("axis", 1)));
    CHECK(p.has("tiles")) << "Number of tiles must be specified";
    tiles_ = static_cast<int>(p.get_int("tiles", 0));
    CHECK_GT(tiles_, 0) << "Number of tiles must be positive.";
    vector<int> top_shape = bottom[0]->shape();
    top_shape[axis] = bottom[0]->shape(axis) * tiles_;
    top[0]->Reshape(top_shape);
    outer_ = bottom[0]->count(0, axis);
    inner_ = bottom[0]->count(axis);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (top[0]->count() == 0) return;
    MC_CHECK(mcTile(bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), outer_, inner_, tiles_,
                    cur_stream()));
  }
  int tiles_ = 0, outer_ = 0, inner_ = 0;
};
REGISTER_LAYER_CLASS(Tile);

// ---------------------------------------------------------------------------
// ShuffleChannel (reference src/layers/shuffle_channel_layer.cpp:9-58; .cu:8-41):
// channels viewed as [group, channels/group] are transposed to
// [channels/group, group].
// ---------------------------------------------------------------------------
class ShuffleChannelLayer : public Layer {
 public:
  explicit ShuffleChannelLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "ShuffleChannel"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    group_ = static_cast<int>(layer_param_.sub("shuffle_channel_param").get_int("group", 1));
    CHECK_GT(group_, 0) << "group must be greater than 0";
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK(bottom[0] != top[0]) << "ShuffleChannel cannot run in place";
    CHECK_EQ(bottom[0]->num_axes(), 4) << "ShuffleChannel takes num x channels x height x width";
    CHECK_EQ(bottom[0]->shape(1) % group_, 0) << "Wrong group size.";
    top[0]->ReshapeLike(*bottom[0]);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Blob& b = *bottom[0];
    if (b.count() == 0) return;
    const int shape[4] = {b.shape(0), group_, b.shape(1) / group_, b.count(2)};
    const int order[4] = {0, 2, 1, 3};
    MC_CHECK(mcPermute(b.gpu_data(), top[0]->mutable_gpu_data(), 4, shape, order, cur_stream()));
  }
  int group_ = 1;
};
REGISTER_LAYER_CLASS(ShuffleChannel);

// ---------------------------------------------------------------------------
// SPP (reference src/layers/spp_layer.cpp:16-199): per pyramid level a Pooling
// layer with 2^level bins per side, flattened and concatenated on axis 1.  The
// bottom is shared by the levels directly (no Split copy).
// ---------------------------------------------------------------------------
class SPPLayer : public Layer {
 public:
  explicit SPPLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "SPP"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("spp_param");
    CHECK(p.has("pyramid_height")) << "pyramid_height must be specified";
    pyramid_height_ = static_cast<int>(p.get_int("pyramid_height", 0));
    CHECK_GT(pyramid_height_, 0) << "pyramid_height must be positive";
    CHECK_LT(pyramid_height_, 16) << "pyramid_height is too large";
    const string pool = p.get_string("pool", "MAX");
    CHECK(pool == "MAX" || pool == "AVE" || pool == "0" || pool == "1")
        << "Unknown pooling method.";
    pool_ = (pool == "AVE" || pool == "1") ? "AVE" : "MAX";
    CHECK(bottom[0] != top[0]) << "SPP cannot run in place";
    pooled_.resize(pyramid_height_);
    flat_.resize(pyramid_height_);
    for (int i = 0; i < pyramid_height_; ++i) {
      pooled_[i].reset(new Blob());
      flat_[i].reset(new Blob());
    }
    built_h_ = built_w_ = -1;
  }

  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_EQ(4, bottom[0]->num_axes())
        << "Input must have 4 axes, corresponding to (num, channels, height, width)";
    const int h = bottom[0]->shape(2), w = bottom[0]->shape(3);
    CHECK_GT(h, 0) << "Input dimensions cannot be zero.";
    CHECK_GT(w, 0) << "Input dimensions cannot be zero.";
    const bool rebuild = h != built_h_ || w != built_w_;
    if (rebuild) {
      pools_.clear();
      flats_.clear();
      for (int i = 0; i < pyramid_height_; ++i) {
        pools_.push_back(LayerRegistry::CreateLayer(PoolingParam(i, h, w)));
        LayerParameter fp;
        fp.set("type", "Flatten", true);
        flats_.push_back(LayerRegistry::CreateLayer(fp));
      }
      LayerParameter cp;
      cp.set("type", "Concat", true);
      concat_ = LayerRegistry::CreateLayer(cp);
      built_h_ = h;
      built_w_ = w;
    }
    if (pyramid_height_ == 1) {
      if (rebuild) pools_[0]->SetUp(bottom, top); else pools_[0]->Reshape(bottom, top);
      return;
    }
    vector<Blob*> flat_ptrs;
    for (int i = 0; i < pyramid_height_; ++i) {
      vector<Blob*> pt(1, pooled_[i].get()), ft(1, flat_[i].get());
      if (rebuild) {
        pools_[i]->SetUp(bottom, pt);
        flats_[i]->SetUp(pt, ft);
      } else {
        pools_[i]->Reshape(bottom, pt);
        flats_[i]->Reshape(pt, ft);
      }
      flat_ptrs.push_back(flat_[i].get());
    }
    if (rebuild) concat_->SetUp(flat_ptrs, top); else concat_->Reshape(flat_ptrs, top);
  }

 protected:
  LayerParameter PoolingParam(int level, int h, int w) const {
    const int bins = 1 << level;
    const int kh = static_cast<int>(std::ceil(h / static_cast<double>(bins)));
    const int kw = static_cast<int>(std::ceil(w / static_cast<double>(bins)));
    LayerParameter lp;
    lp.set("type", "Pooling", true);
    Message* pp = lp.add_sub("pooling_param");
    pp->set("pool", pool_);
    pp->add_int("pad_h", (kh * bins - h + 1) / 2);
    pp->add_int("pad_w", (kw * bins - w + 1) / 2);
    pp->add_int("kernel_h", kh);
    pp->add_int("kernel_w", kw);
    pp->add_int("stride_h", kh);
    pp->add_int("stride_w", kw);
    return lp;
  }

  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (pyramid_height_ == 1) {
      pools_[0]->Forward(bottom, top);
      return;
    }
    vector<Blob*> flat_ptrs;
    for (int i = 0; i < pyramid_height_; ++i) {
      vector<Blob*> pt(1, pooled_[i].get()), ft(1, flat_[i].get());
      pools_[i]->Forward(bottom, pt);
      flats_[i]->Forward(pt, ft);
      flat_ptrs.push_back(flat_[i].get());
    }
    concat_->Forward(flat_ptrs, top);
  }

  int pyramid_height_ = 0, built_h_ = -1, built_w_ = -1;
  string pool_;
  vector<shared_ptr<Layer> > pools_, flats_;
  shared_ptr<Layer> concat_;
  vector<shared_ptr<Blob> > pooled_, flat_;
};
REGISTER_LAYER_CLASS(SPP);

// ---------------------------------------------------------------------------
// Parameter (reference src/layers/parameter_layer.hpp:10-36, .cpp:6-14): a
// learned blob published as a top.
// ---------------------------------------------------------------------------
class ParameterLayer : public Layer {
 public:
  explicit ParameterLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Parameter"; }
  int ExactNumBottomBlobs() const override { return 0; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& shape = layer_param_.sub("parameter_param").sub("shape");
    vector<int> dims;
    for (int i = 0; i < shape.count("dim"); ++i)
      dims.push_back(static_cast<int>(shape.get_int("dim", 0, i)));
    if (blobs_.empty()) {
      blobs_.resize(1);
      blobs_[0].reset(new Blob(dims));
      Message zero;
      FillConstant(zero, blobs_[0].get());
    }
    top[0]->Reshape(dims);
    CHECK_EQ(top[0]->count(), blobs_[0]->count()) << "Parameter blob and shape differ";
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {}

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    DeviceCopy(*blobs_[0], top[0]);
  }
};
REGISTER_LAYER_CLASS(Parameter);

}  // namespace caffe
