// Layout layers: Concat, Slice, Flatten, Reshape, Permute, Split, plus
// Normalize and PriorBox from the SSD graph.
#include <algorithm>
#include <cmath>

#include "layer.hpp"

namespace caffe {

// ---------------------------------------------------------------------------
// Concat (reference src/layers/concat_layer.cpp:8-70; .cu:8-46)
// ---------------------------------------------------------------------------
class ConcatLayer : public Layer {
 public:
  explicit ConcatLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Concat"; }
  int MinBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }
  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("concat_param");
    CHECK(!(p.has("axis") && p.has("concat_dim")))
        << "Either axis or concat_dim should be specified; not both.";
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("concat_param");
    const int num_axes = bottom[0]->num_axes();
    if (p.has("concat_dim")) {
      axis_ = static_cast<int>(p.get_int("concat_dim"));
      CHECK_GE(axis_, 0) << "concat_dim must be non-negative";
      CHECK_LT(axis_, num_axes) << "concat_dim out of range.";
    } else {
      axis_ = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("axis", 1)));
    }
    vector<int> top_shape = bottom[0]->shape();
    outer_ = bottom[0]->count(0, axis_);
    inner_ = bottom[0]->count(axis_ + 1);
    long sum = bottom[0]->count();
    for (size_t i = 1; i < bottom.size(); ++i) {
      CHECK_EQ(num_axes, bottom[i]->num_axes()) << "All inputs must have the same #axes.";
      for (int j = 0; j < num_axes; ++j) {
        if (j == axis_) continue;
        CHECK_EQ(top_shape[j], bottom[i]->shape(j))
            << "All inputs must have the same shape, except at concat_axis.";
      }
      sum += bottom[i]->count();
      top_shape[axis_] += bottom[i]->shape(axis_);
    }
    top[0]->Reshape(top_shape);
    CHECK_EQ(sum, static_cast<long>(top[0]->count()));
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom.size() == 1) {
      DeviceCopy(*bottom[0], top[0]);
      return;
    }
    // all bottoms in one launch (per eight of them)
    vector<const float*> srcs;
    vector<long> widths;
    for (Blob* b : bottom) {
      srcs.push_back(b->gpu_data());
      widths.push_back(static_cast<long>(b->shape(axis_)) * inner_);
    }
    MC_CHECK(mcConcat(srcs.data(), widths.data(), static_cast<int>(srcs.size()),
                      top[0]->mutable_gpu_data(), outer_, cur_stream()));
  }
  int axis_ = 1, outer_ = 0, inner_ = 0;
};
REGISTER_LAYER_CLASS(Concat);

// ---------------------------------------------------------------------------
// Slice (reference src/layers/slice_layer.cpp:8-110; .cu:8-46)
// ---------------------------------------------------------------------------
class SliceLayer : public Layer {
 public:
  explicit SliceLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Slice"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int MinTopBlobs() const override { return 1; }
  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("slice_param");
    CHECK(!(p.has("axis") && p.has("slice_dim")))
        << "Either axis or slice_dim should be specified; not both.";
    points_.clear();
    for (int i = 0; i < p.count("slice_point"); ++i)
      points_.push_back(static_cast<int>(p.get_int("slice_point", 0, i)));
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("slice_param");
    const int num_axes = bottom[0]->num_axes();
    if (p.has("slice_dim")) {
      axis_ = static_cast<int>(p.get_int("slice_dim"));
      CHECK_GE(axis_, 0) << "slice_dim must be non-negative";
      CHECK_LT(axis_, num_axes) << "slice_dim out of range.";
    } else {
      axis_ = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("axis", 1)));
    }
    vector<int> top_shape = bottom[0]->shape();
    const int extent = bottom[0]->shape(axis_);
    outer_ = bottom[0]->count(0, axis_);
    inner_ = bottom[0]->count(axis_ + 1);
    long count = 0;
    if (!points_.empty()) {
      CHECK_EQ(points_.size(), top.size() - 1);
      CHECK_LE(static_cast<int>(top.size()), extent);
      int prev = 0;
      vector<int> slices;
      for (int pt : points_) {
        CHECK_GT(pt, prev);
        slices.push_back(pt - prev);
        prev = pt;
      }
      slices.push_back(extent - prev);
      for (size_t i = 0; i < top.size(); ++i) {
        top_shape[axis_] = slices[i];
        top[i]->Reshape(top_shape);
        count += top[i]->count();
      }
    } else {
      CHECK_EQ(extent % static_cast<int>(top.size()), 0)
          << "Number of top blobs (" << top.size() << ") should evenly divide input slice axis ("
          << extent << ")";
      top_shape[axis_] = extent / static_cast<int>(top.size());
      for (Blob* t : top) {
        t->Reshape(top_shape);
        count += t->count();
      }
    }
    CHECK_EQ(count, static_cast<long>(bottom[0]->count()));
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (top.size() == 1) {
      DeviceCopy(*bottom[0], top[0]);
      return;
    }
    const float* bottom_data = bottom[0]->gpu_data();
    const long bottom_pitch = static_cast<long>(bottom[0]->shape(axis_)) * inner_;
    long offset = 0;
    for (Blob* t : top) {
      const long width = static_cast<long>(t->shape(axis_)) * inner_;
      if (width > 0 && outer_ > 0)
        MC_CHECK(mcCopy2D(bottom_data + offset, bottom_pitch, t->mutable_gpu_data(), width, width,
                          outer_, cur_stream()));
      offset += width;
    }
  }
  int axis_ = 1, outer_ = 0, inner_ = 0;
  vector<int> points_;
};
REGISTER_LAYER_CLASS(Slice);

// ---------------------------------------------------------------------------
// Flatten / Reshape / Split: shape-only (reference flatten_layer.cpp:8-39,
// reshape_layer.cpp:8-105, split_layer.cpp:8-45); data moves with one copy
// unless the layer runs in place.
// ---------------------------------------------------------------------------
class FlattenLayer : public Layer {
 public:
  explicit FlattenLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Flatten"; }
  bool IsView() const override { return true; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("flatten_param");
    const int start = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("axis", 1)));
    const int end = bottom[0]->CanonicalAxisIndex(static_cast<int>(p.get_int("end_axis", -1)));
    vector<int> top_shape(bottom[0]->shape().begin(), bottom[0]->shape().begin() + start);
    top_shape.push_back(bottom[0]->count(start, end + 1));
    for (int i = end + 1; i < bottom[0]->num_axes(); ++i) top_shape.push_back(bottom[0]->shape(i));
    const int count = bottom[0]->count();
    top[0]->Reshape(top_shape);
    CHECK_EQ(top[0]->count(), count);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom[0] == top[0]) return;
    // the bottom's producer may have given it its final shape in its own Forward
    if (bottom[0]->count() != top[0]->count()) Reshape(bottom, top);
    DeviceCopy(*bottom[0], top[0]);
  }
};
REGISTER_LAYER_CLASS(Flatten);

class ReshapeLayer : public Layer {
 public:
  explicit ReshapeLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Reshape"; }
  bool IsView() const override { return true; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }
  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_NE(top[0], bottom[0]) << type() << " Layer does not allow in-place computation.";
    const Message& shape = layer_param_.sub("reshape_param").sub("shape");
    dims_.clear();
    copy_axes_.clear();
    inferred_axis_ = -1;
    constant_count_ = 1;
    for (int i = 0; i < shape.count("dim"); ++i) {
      const int d = static_cast<int>(shape.get_int("dim", 0, i));
      dims_.push_back(d);
      if (d == 0) {
        copy_axes_.push_back(i);
      } else if (d == -1) {
        CHECK_EQ(inferred_axis_, -1) << "new shape contains multiple -1 dims; at most a single "
                                     << "(1) value of -1 may be specified";
        inferred_axis_ = i;
      } else {
        constant_count_ *= d;
      }
    }
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("reshape_param");
    const int in_axis = static_cast<int>(p.get_int("axis", 0));
    const int nb = bottom[0]->num_axes();
    const int start = in_axis >= 0 ? in_axis : nb + in_axis + 1;
    CHECK_GE(start, 0) << "axis " << in_axis << " out of range";
    CHECK_LE(start, nb) << "axis " << in_axis << " out of range for " << nb << "-D input blob";
    const int num_axes = static_cast<int>(p.get_int("num_axes", -1));
    CHECK_GE(num_axes, -1) << "num_axes must be >= 0, or -1 for all";
    const int end = num_axes == -1 ? nb : start + num_axes;
    CHECK_LE(end, nb) << "end_axis = axis + num_axes is out of range";
    vector<int> top_shape(bottom[0]->shape().begin(), bottom[0]->shape().begin() + start);
    top_shape.insert(top_shape.end(), dims_.begin(), dims_.end());
    top_shape.insert(top_shape.end(), bottom[0]->shape().begin() + end, bottom[0]->shape().end());
    for (int a : copy_axes_) {
      CHECK_GT(nb, start + a) << "new shape contains a 0, but there was no corresponding bottom "
                              << "axis to copy";
      top_shape[start + a] = bottom[0]->shape(start + a);
    }
    if (inferred_axis_ >= 0) {
      int explicit_count = constant_count_ * bottom[0]->count(0, start) * bottom[0]->count(end);
      for (int a : copy_axes_) explicit_count *= top_shape[start + a];
      CHECK_GT(explicit_count, 0) << "cannot infer a dimension of an empty blob";
      CHECK_EQ(0, bottom[0]->count() % explicit_count)
          << "bottom count (" << bottom[0]->count() << ") must be divisible by the product of "
          << "the specified dimensions (" << explicit_count << ")";
      top_shape[start + inferred_axis_] = bottom[0]->count() / explicit_count;
    }
    top[0]->Reshape(top_shape);
    CHECK_EQ(top[0]->count(), bottom[0]->count()) << "output count must match input count";
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    // the bottom's producer may have given it its final shape in its own Forward
    if (bottom[0]->count() != top[0]->count()) Reshape(bottom, top);
    DeviceCopy(*bottom[0], top[0]);
  }
  vector<int> dims_, copy_axes_;
  int inferred_axis_ = -1, constant_count_ = 1;
};
REGISTER_LAYER_CLASS(Reshape);

class SplitLayer : public Layer {
 public:
  explicit SplitLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Split"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int MinTopBlobs() const override { return 1; }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    for (Blob* t : top) {
      CHECK_NE(t, bottom[0]) << type() << " Layer does not allow in-place computation.";
      t->ReshapeLike(*bottom[0]);
    }
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    for (Blob* t : top) DeviceCopy(*bottom[0], t);
  }
};
REGISTER_LAYER_CLASS(Split);

// ---------------------------------------------------------------------------
// Permute (reference src/layers/permute_layer.cpp:9-106; .cu:10-51)
// ---------------------------------------------------------------------------
class PermuteLayer : public Layer {
 public:
  explicit PermuteLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Permute"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }
  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("permute_param");
    num_axes_ = bottom[0]->num_axes();
    CHECK_LE(num_axes_, 8) << "Permute supports at most 8 axes";
    order_.clear();
    for (int i = 0; i < p.count("order"); ++i) {
      const int o = static_cast<int>(p.get_int("order", 0, i));
      CHECK_LT(o, num_axes_) << "order should be less than the input dimension.";
      CHECK_GE(o, 0) << "order must be non-negative";
      if (std::find(order_.begin(), order_.end(), o) != order_.end())
        LOG(FATAL) << "there are duplicate orders";
      order_.push_back(o);
    }
    // axes not named keep their relative order at the end
    for (int i = 0; i < num_axes_; ++i)
      if (std::find(order_.begin(), order_.end(), i) == order_.end()) order_.push_back(i);
    CHECK_EQ(num_axes_, static_cast<int>(order_.size()));
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_EQ(bottom[0]->num_axes(), num_axes_) << "bottom num_axes may not change.";
    vector<int> top_shape;
    for (int i = 0; i < num_axes_; ++i) top_shape.push_back(bottom[0]->shape(order_[i]));
    CHECK_NE(top[0], bottom[0]) << "Permute Layer does not allow in-place computation.";
    top[0]->Reshape(top_shape);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    if (bottom[0]->count() == 0) return;
    MC_CHECK(mcPermute(bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), num_axes_,
                       bottom[0]->shape().data(), order_.data(), cur_stream()));
  }
  int num_axes_ = 0;
  vector<int> order_;
};
REGISTER_LAYER_CLASS(Permute);

// ---------------------------------------------------------------------------
// Normalize (reference src/layers/normalize_layer.cpp:8-135; .cu:15-103)
// ---------------------------------------------------------------------------
class NormalizeLayer : public Layer {
 public:
  explicit NormalizeLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "Normalize"; }
  int ExactNumBottomBlobs() const override { return 1; }
  int ExactNumTopBlobs() const override { return 1; }
  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_GE(bottom[0]->num_axes(), 2) << "Number of axes of bottom blob must be >=2.";
    const Message& p = layer_param_.sub("norm_param");
    across_spatial_ = p.get_bool("across_spatial", true);
    channel_shared_ = p.get_bool("channel_shared", true);
    eps_ = static_cast<float>(p.get_float("eps", 1e-10));
    const int channels = bottom[0]->channels();
    if (blobs_.empty()) {
      blobs_.resize(1);
      blobs_[0].reset(new Blob(channel_shared_ ? vector<int>() : vector<int>{channels}));
      const real_t v = p.has("scale_filler")
                           ? static_cast<real_t>(p.sub("scale_filler").get_float("value", 0.))
                           : 1.f;
      real_t* d = blobs_[0]->mutable_cpu_data();
      for (int i = 0; i < blobs_[0]->count(); ++i) d[i] = v;
    }
    CHECK_EQ(blobs_[0]->count(), channel_shared_ ? 1 : channels)
        << "Scale size is inconsistent with prototxt config";
  }
  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    CHECK_GE(bottom[0]->num_axes(), 2) << "Number of axes of bottom blob must be >=2.";
    top[0]->ReshapeLike(*bottom[0]);
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    MC_CHECK(mcNormalize(bottom[0]->gpu_data(), top[0]->mutable_gpu_data(), bottom[0]->num(),
                         bottom[0]->channels(), bottom[0]->height() * bottom[0]->width(),
                         across_spatial_ ? 1 : 0, channel_shared_ ? 1 : 0, eps_,
                         blobs_[0]->gpu_data(), cur_stream()));
  }
  bool across_spatial_ = true, channel_shared_ = true;
  float eps_ = 1e-10f;
};
REGISTER_LAYER_CLASS(Normalize);

// ---------------------------------------------------------------------------
// PriorBox (reference src/layers/prior_box_layer.cpp:11-217).  The table
// depends on shapes and layer parameters only, never on blob contents; the
// reference computes it on the host in GPU mode too (it has no device code), and
// so does this layer: once per shape, then the result lives on the device.
// The float/double mix of the reference's expressions is kept literally.
// ---------------------------------------------------------------------------
class PriorBoxLayer : public Layer {
 public:
  explicit PriorBoxLayer(const LayerParameter& param) : Layer(param) {}
  const char* type() const override { return "PriorBox"; }
  int ExactNumBottomBlobs() const override { return 2; }
  int ExactNumTopBlobs() const override { return 1; }

  void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const Message& p = layer_param_.sub("prior_box_param");
    CHECK_GT(p.count("min_size"), 0) << "must provide min_size.";
    for (int i = 0; i < p.count("min_size"); ++i) {
      min_sizes_.push_back(static_cast<float>(p.get_float("min_size", 0., i)));
      CHECK_GT(min_sizes_.back(), 0) << "min_size must be positive.";
    }
    aspect_ratios_.assign(1, 1.f);
    flip_ = p.get_bool("flip", true);
    for (int i = 0; i < p.count("aspect_ratio"); ++i) {
      const float ar = static_cast<float>(p.get_float("aspect_ratio", 0., i));
      bool already = false;
      for (float a : aspect_ratios_) already = already || std::fabs(ar - a) < 1e-6;
      if (!already) {
        aspect_ratios_.push_back(ar);
        if (flip_) aspect_ratios_.push_back(static_cast<float>(1. / ar));
      }
    }
    num_priors_ = static_cast<int>(aspect_ratios_.size() * min_sizes_.size());
    if (p.count("max_size") > 0) {
      CHECK_EQ(p.count("min_size"), p.count("max_size"));
      for (int i = 0; i < p.count("max_size"); ++i) {
        max_sizes_.push_back(static_cast<float>(p.get_float("max_size", 0., i)));
        CHECK_GT(max_sizes_[i], min_sizes_[i]) << "max_size must be greater than min_size.";
        num_priors_ += 1;
      }
    }
    clip_ = p.get_bool("clip", false);
    const int nv = p.count("variance");
    if (nv > 1) {
      CHECK_EQ(nv, 4);
      for (int i = 0; i < 4; ++i) {
        variance_.push_back(static_cast<float>(p.get_float("variance", 0., i)));
        CHECK_GT(variance_.back(), 0);
      }
    } else if (nv == 1) {
      variance_.push_back(static_cast<float>(p.get_float("variance")));
      CHECK_GT(variance_.back(), 0);
    } else {
      variance_.push_back(0.1f);
    }
    if (p.has("img_h") || p.has("img_w")) {
      CHECK(!p.has("img_size")) << "Either img_size or img_h/img_w should be specified; not both.";
      img_h_ = static_cast<int>(p.get_int("img_h", 0));
      img_w_ = static_cast<int>(p.get_int("img_w", 0));
      CHECK_GT(img_h_, 0) << "img_h should be larger than 0.";
      CHECK_GT(img_w_, 0) << "img_w should be larger than 0.";
    } else if (p.has("img_size")) {
      img_h_ = img_w_ = static_cast<int>(p.get_int("img_size"));
      CHECK_GT(img_h_, 0) << "img_size should be larger than 0.";
    }
    if (p.has("step_h") || p.has("step_w")) {
      CHECK(!p.has("step")) << "Either step or step_h/step_w should be specified; not both.";
      step_h_ = static_cast<float>(p.get_float("step_h", 0.));
      step_w_ = static_cast<float>(p.get_float("step_w", 0.));
      CHECK_GT(step_h_, 0.) << "step_h should be larger than 0.";
      CHECK_GT(step_w_, 0.) << "step_w should be larger than 0.";
    } else if (p.has("step")) {
      step_h_ = step_w_ = static_cast<float>(p.get_float("step"));
      CHECK_GT(step_h_, 0) << "step should be larger than 0.";
    }
    offset_ = static_cast<float>(p.get_float("offset", 0.5));
  }

  void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const int dim = bottom[0]->width() * bottom[0]->height() * num_priors_ * 4;
    CHECK_GT(dim, 0);
    top[0]->Reshape(vector<int>{1, 2, dim});
  }

 protected:
  void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) override {
    const int lw = bottom[0]->width(), lh = bottom[0]->height();
    const int iw = (img_h_ == 0 || img_w_ == 0) ? bottom[1]->width() : img_w_;
    const int ih = (img_h_ == 0 || img_w_ == 0) ? bottom[1]->height() : img_h_;
    const vector<int> key = {lw, lh, iw, ih};
    if (key != cached_key_) {
      Compute(lw, lh, iw, ih);
      cached_key_ = key;
    }
    // the net may have recycled the top's memory: refresh it from the cached table
    MC_CHECK(mcCopy2D(table_.gpu_data(), table_.count(), top[0]->mutable_gpu_data(),
                      table_.count(), table_.count(), 1, cur_stream()));
  }

  void Compute(int layer_width, int layer_height, int img_width, int img_height) {
    float step_w, step_h;
    if (step_w_ == 0 || step_h_ == 0) {
      step_w = static_cast<float>(img_width) / layer_width;
      step_h = static_cast<float>(img_height) / layer_height;
    } else {
      step_w = step_w_;
      step_h = step_h_;
    }
    const int dim = layer_height * layer_width * num_priors_ * 4;
    table_.Reshape(vector<int>{1, 2, dim});
    real_t* out = table_.mutable_cpu_data();
    int idx = 0;
    auto emit = [&](float cx, float cy, float bw, float bh) {
      out[idx++] = static_cast<real_t>((cx - bw / 2.) / img_width);
      out[idx++] = static_cast<real_t>((cy - bh / 2.) / img_height);
      out[idx++] = static_cast<real_t>((cx + bw / 2.) / img_width);
      out[idx++] = static_cast<real_t>((cy + bh / 2.) / img_height);
    };
    for (int h = 0; h < layer_height; ++h) {
      for (int w = 0; w < layer_width; ++w) {
        const float center_x = (w + offset_) * step_w;
        const float center_y = (h + offset_) * step_h;
        for (size_t s = 0; s < min_sizes_.size(); ++s) {
          const int min_size = static_cast<int>(min_sizes_[s]);  // the reference truncates
          float bw = static_cast<float>(min_size), bh = bw;
          emit(center_x, center_y, bw, bh);
          if (!max_sizes_.empty()) {
            const int max_size = static_cast<int>(max_sizes_[s]);
            bw = bh = static_cast<float>(std::sqrt(static_cast<double>(min_size * max_size)));
            emit(center_x, center_y, bw, bh);
          }
          for (float ar : aspect_ratios_) {
            if (std::fabs(ar - 1.) < 1e-6) continue;
            bw = min_size * sqrtf(ar);
            bh = min_size / sqrtf(ar);
            emit(center_x, center_y, bw, bh);
          }
        }
      }
    }
    CHECK_EQ(idx, dim);
    if (clip_)
      for (int d = 0; d < dim; ++d) out[d] = std::min<real_t>(std::max<real_t>(out[d], 0.f), 1.f);
    real_t* var = out + dim;
    if (variance_.size() == 1) {
      for (int d = 0; d < dim; ++d) var[d] = variance_[0];
    } else {
      for (int d = 0; d < dim; ++d) var[d] = variance_[d % 4];
    }
  }

  vector<float> min_sizes_, max_sizes_, aspect_ratios_, variance_;
  bool flip_ = true, clip_ = false;
  int num_priors_ = 0, img_w_ = 0, img_h_ = 0;
  float step_w_ = 0.f, step_h_ = 0.f, offset_ = 0.5f;
  Blob table_;
  vector<int> cached_key_;
};
REGISTER_LAYER_CLASS(PriorBox);

}  // namespace caffe
