// Layer: the operator plug-in interface of the forward path, and its registry.
//
// Same contract as the reference's src/layer.hpp:25-279 and
// src/layer_factory.hpp:54-127: a layer is constructed from its LayerParameter
// (taking over any blobs stored there), SetUp = CheckBlobCounts + LayerSetUp +
// Reshape, Forward dispatches on the calling thread's mode, and layer classes
// register a creator under their prototxt `type:` string at static-init time.
//
// Differences, on purpose: Forward_gpu is the one implementation every layer
// must provide; Forward_cpu is not implemented in this library and raises.
// Layers that transform a blob per channel, in place, can describe themselves as
// an epilogue stage so that Net can fold them into the preceding contraction.
#ifndef MCHIP_RUNTIME_LAYER_HPP_
#define MCHIP_RUNTIME_LAYER_HPP_

#include <map>
#include <string>
#include <vector>

#include "caffe/blob.hpp"
#include "device.hpp"
#include "mchip/kernels.h"
#include "proto.hpp"

namespace caffe {

class Layer {
 public:
  explicit Layer(const LayerParameter& param) : layer_param_(param) {
    // Blobs stored with the layer definition become its parameters.
    for (const auto& f : param.fields()) {
      if (f.name == "blobs" && f.msg) {
        shared_ptr<Blob> b(new Blob());
        b->FromProto(static_cast<const BlobProto&>(*f.msg));
        blobs_.push_back(b);
      }
    }
  }
  virtual ~Layer() {}

  void SetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) {
    CheckBlobCounts(bottom, top);
    LayerSetUp(bottom, top);
    Reshape(bottom, top);
  }

  virtual void LayerSetUp(const vector<Blob*>& bottom, const vector<Blob*>& top) {}
  virtual void Reshape(const vector<Blob*>& bottom, const vector<Blob*>& top) = 0;

  inline void Forward(const vector<Blob*>& bottom, const vector<Blob*>& top) {
    switch (Context::mode()) {
      case CPU:
        Forward_cpu(bottom, top);
        break;
      case GPU:
        Forward_gpu(bottom, top);
        break;
      default:
        LOG(FATAL) << "Unknown caffe mode.";
    }
  }

  vector<shared_ptr<Blob> >& blobs() { return blobs_; }
  const LayerParameter& layer_param() const { return layer_param_; }
  // The layer's definition with its current parameter blobs in place of the ones
  // it was built from (reference src/layer.hpp:282-289).
  void ToProto(LayerParameter* param) const {
    *param = layer_param_;
    param->remove("blobs");
    for (const auto& b : blobs_) b->ToProto(static_cast<BlobProto*>(param->add_sub("blobs")));
  }
  const string name() const { return layer_param_.get_string("name"); }

  virtual const char* type() const { return ""; }
  virtual int ExactNumBottomBlobs() const { return -1; }
  virtual int MinBottomBlobs() const { return -1; }
  virtual int MaxBottomBlobs() const { return -1; }
  virtual int ExactNumTopBlobs() const { return -1; }
  virtual int MinTopBlobs() const { return -1; }
  virtual int MaxTopBlobs() const { return -1; }
  virtual bool EqualNumBottomTopBlobs() const { return false; }

  // Scratch blobs whose memory Net may share with dead activations.
  virtual vector<Blob*> GetTempBlobs() { return vector<Blob*>(); }

  // ---- epilogue folding (no counterpart in the reference) -------------------
  // True when this layer, running in place on a blob with `channels` channels
  // on axis 1, is one per-channel stage (sub/div/mul/add then activation).
  virtual bool IsChannelStage(int channels) const { return false; }
  // Device pointers of the stage for the current parameters; may launch small
  // preparatory kernels on the thread's stream.
  virtual void GetChannelStage(mcChannelOp* op) { LOG(FATAL) << type() << ": not a channel stage"; }
  // Changes whenever the stage's parameters may have changed.
  virtual uint64_t ChannelStageVersion() const { return 0; }
  // True when this layer can absorb following channel stages into its kernel.
  virtual bool AcceptsEpilogue() const { return false; }
  // How many non-activation stages it can absorb (an activation may follow them).
  virtual int MaxAffineFollowers() const { return 0; }
  // Whether `follower` (already known to be an in-place channel stage) may ride
  // along; a layer whose own pass fixes some fields of the stage refuses
  // followers that need those fields.
  virtual bool AcceptsFollower(const Layer* follower) const { return true; }
  virtual void SetEpilogue(const vector<Layer*>& followers) {}
  // Residual folding.  A two-input sum with unit coefficients reports itself
  // (and the activation it absorbed, if any) so that the layer producing one of
  // its inputs can add the other in its own epilogue and the sum never runs.
  virtual bool IsPlainSum() const { return false; }
  virtual Layer* AbsorbedActivation() const { return nullptr; }
  // True when the layer's epilogue can still take `+ residual` and an
  // activation (its own followers end without an activation).
  virtual bool AcceptsResidual() const { return false; }
  virtual void SetResidual(Blob* residual, Layer* activation) {}
  // Sibling merge.  Two Convolution layers that read the same blob with the same
  // window geometry, with nothing folded into either, can run as one launch over
  // the concatenated filters (the loc and conf heads of an SSD source).  A layer
  // that could take part describes its geometry in `key`; the first of a pair
  // adopts the second, computes both tops in its own Forward, and the second is
  // skipped.  AdoptSibling(nullptr, nullptr) ends the arrangement.
  virtual bool SiblingKey(vector<int>* key) const { return false; }
  virtual void AdoptSibling(Layer* sibling, Blob* sibling_top) {}
  // True when the top holds the bottom's values in the same order under another
  // shape (Flatten, Reshape).  When nothing reads the bottom afterwards Net lets
  // the top take over the bottom's memory and skips the layer's copy.
  virtual bool IsView() const { return false; }
  // True when Forward gives a top a shape (and possibly new memory) that is only
  // known after the device has run (DetectionOutput's row count).  Such a top
  // cannot be aliased by a view that was placed before Forward.
  virtual bool ShapesTopInForward() const { return false; }

 protected:
  LayerParameter layer_param_;
  vector<shared_ptr<Blob> > blobs_;

  virtual void Forward_cpu(const vector<Blob*>& bottom, const vector<Blob*>& top) {
    LOG(FATAL) << "layer '" << name() << "' (" << type()
               << "): this library implements the HIP device path only; call "
               << "SetMode(GPU, device) before Forward";
  }
  virtual void Forward_gpu(const vector<Blob*>& bottom, const vector<Blob*>& top) = 0;

  virtual void CheckBlobCounts(const vector<Blob*>& bottom, const vector<Blob*>& top) {
    const int nb = static_cast<int>(bottom.size()), nt = static_cast<int>(top.size());
    if (ExactNumBottomBlobs() >= 0)
      CHECK_EQ(ExactNumBottomBlobs(), nb)
          << type() << " Layer takes " << ExactNumBottomBlobs() << " bottom blob(s) as input.";
    if (MinBottomBlobs() >= 0)
      CHECK_LE(MinBottomBlobs(), nb)
          << type() << " Layer takes at least " << MinBottomBlobs() << " bottom blob(s) as input.";
    if (MaxBottomBlobs() >= 0)
      CHECK_GE(MaxBottomBlobs(), nb)
          << type() << " Layer takes at most " << MaxBottomBlobs() << " bottom blob(s) as input.";
    if (ExactNumTopBlobs() >= 0)
      CHECK_EQ(ExactNumTopBlobs(), nt)
          << type() << " Layer produces " << ExactNumTopBlobs() << " top blob(s) as output.";
    if (MinTopBlobs() >= 0)
      CHECK_LE(MinTopBlobs(), nt)
          << type() << " Layer produces at least " << MinTopBlobs() << " top blob(s) as output.";
    if (MaxTopBlobs() >= 0)
      CHECK_GE(MaxTopBlobs(), nt)
          << type() << " Layer produces at most " << MaxTopBlobs() << " top blob(s) as output.";
    if (EqualNumBottomTopBlobs())
      CHECK_EQ(nb, nt) << type() << " Layer produces one top blob as output for each bottom "
                       << "blob input.";
  }

  DISABLE_COPY_AND_ASSIGN(Layer);
};

class LayerRegistry {
 public:
  typedef shared_ptr<Layer> (*Creator)(const LayerParameter&);
  typedef std::map<string, Creator> CreatorRegistry;

  static CreatorRegistry& Registry() {
    static CreatorRegistry* g_registry = new CreatorRegistry();
    return *g_registry;
  }
  static void AddCreator(const string& type, Creator creator) {
    CreatorRegistry& registry = Registry();
    CHECK_EQ(registry.count(type), 0u) << "Layer type " << type << " already registered.";
    registry[type] = creator;
  }
  static shared_ptr<Layer> CreateLayer(const LayerParameter& param) {
    const string type = param.get_string("type");
    CreatorRegistry& registry = Registry();
    if (registry.count(type) == 0) {
      string known;
      for (auto& kv : registry) known += (known.empty() ? "" : ", ") + kv.first;
      LOG(FATAL) << "Unknown layer type: " << type << " (known types: " << known << ")";
    }
    return registry[type](param);
  }
  static vector<string> LayerTypeList() {
    vector<string> types;
    for (auto& kv : Registry()) types.push_back(kv.first);
    return types;
  }

 private:
  LayerRegistry() {}
};

class LayerRegisterer {
 public:
  LayerRegisterer(const string& type, LayerRegistry::Creator creator) {
    LayerRegistry::AddCreator(type, creator);
  }
};

#define REGISTER_LAYER_CREATOR(type, creator) \
  static ::caffe::LayerRegisterer g_creator_##type(#type, creator)

#define REGISTER_LAYER_CLASS(type)                                          \
  static shared_ptr<Layer> Creator_##type##Layer(const LayerParameter& p) { \
    return shared_ptr<Layer>(new type##Layer(p));                           \
  }                                                                         \
  REGISTER_LAYER_CREATOR(type, Creator_##type##Layer)

// Every filler type fills with FillerParameter.value (default 0), as in the
// reference (src/filler.hpp:28-71).
inline void FillConstant(const Message& filler, Blob* blob, double default_value = 0.) {
  const string type = filler.get_string("type", "constant");
  static const char* kKnown[] = {"constant", "gaussian", "positive_unitball", "uniform",
                                 "xavier",   "msra",     "bilinear"};
  bool known = false;
  for (const char* k : kKnown) known = known || type == k;
  CHECK(known) << "Unknown filler name: " << type;
  const real_t value = static_cast<real_t>(filler.get_float("value", default_value));
  real_t* data = blob->mutable_cpu_data();
  for (int i = 0; i < blob->count(); ++i) data[i] = value;
}

// Changes whenever the blob's memory may have been written.
inline uint64_t BlobVersion(const shared_ptr<Blob>& b) {
  return b && b->data() ? b->data()->version() : 0;
}

// Device-to-device copy of a whole blob on the calling thread's stream.
inline void DeviceCopy(const Blob& src, Blob* dst) {
  if (src.count() == 0) return;
  MC_CHECK(mcCopy2D(src.gpu_data(), src.count(), dst->mutable_gpu_data(), src.count(),
                    src.count(), 1, Context::Get().stream()));
}

// Stream of the calling thread, as the void* the kernel ABI takes.
inline void* cur_stream() { return Context::Get().stream(); }

}  // namespace caffe

#endif  // MCHIP_RUNTIME_LAYER_HPP_
