#include "caffe/net.hpp"

#include <algorithm>
#include <sstream>

#include "caffe/profiler.hpp"
#include "layer.hpp"
#include "proto.hpp"

namespace caffe {

namespace {
// The idx-th `layer { }` entry of a NetParameter.
const LayerParameter& LayerAt(const NetParameter& param, int idx) {
  return static_cast<const LayerParameter&>(param.sub("layer", idx));
}
}  // namespace

Net::Net(const string& param_file) {
  NetParameter param;
  ReadNetParamsFromTextFileOrDie(param_file, &param);
  Init(param);
}

Net::~Net() {
  // Kernels of the last Forward may still be reading the blobs being released.
  if (Context::gpu_available() && Context::mode() == GPU) {
    try {
      Context::Get().Sync();
    } catch (...) {
    }
  }
}

// Builds every layer and wires bottoms/tops by blob name, as the reference's
// Net::Init does (reference src/net.cpp:26-73).
void Net::Init(const NetParameter& param) {
  name_ = param.get_string("name");
  std::map<string, int> blob_name_to_idx;
  std::set<string> available_blobs;
  const int n_layers = param.count("layer");
  CHECK_GT(n_layers, 0) << "network has no layers";
  bottom_vecs_.resize(n_layers);
  top_vecs_.resize(n_layers);
  bottom_id_vecs_.resize(n_layers);
  top_id_vecs_.resize(n_layers);
  param_id_vecs_.resize(n_layers);
  for (int layer_id = 0; layer_id < n_layers; ++layer_id) {
    const LayerParameter& layer_param = LayerAt(param, layer_id);
    layers_.push_back(LayerRegistry::CreateLayer(layer_param));
    layer_names_.push_back(layer_param.get_string("name"));
    for (int b = 0; b < layer_param.count("bottom"); ++b)
      AppendBottom(param, layer_id, b, &available_blobs, &blob_name_to_idx);
    for (int t = 0; t < layer_param.count("top"); ++t)
      AppendTop(param, layer_id, t, &available_blobs, &blob_name_to_idx);
    layers_[layer_id]->SetUp(bottom_vecs_[layer_id], top_vecs_[layer_id]);
    const int num_param_blobs = static_cast<int>(layers_[layer_id]->blobs().size());
    for (int p = 0; p < num_param_blobs; ++p) AppendParam(param, layer_id, p);
  }
  CHECK_EQ(std::string(layers_[0]->type()), std::string("Input"))
      << "Network's first layer should be Input Layer.";
  // Inputs stay valid for the whole forward pass.
  for (int blob_id : top_id_vecs_[0]) blob_life_time_[blob_id] = static_cast<int>(layers_.size());
  for (size_t blob_id = 0; blob_id < blob_names_.size(); ++blob_id) {
    blob_names_index_[blob_names_[blob_id]] = static_cast<int>(blob_id);
    blobs_[blob_id]->set_name(blob_names_[blob_id]);
  }
  for (size_t layer_id = 0; layer_id < layer_names_.size(); ++layer_id)
    layer_names_index_[layer_names_[layer_id]] = static_cast<int>(layer_id);
  layer_fused_.assign(layers_.size(), 0);
  sibling_owner_.assign(layers_.size(), -1);
  residual_alias_.assign(layers_.size(), -1);
  PlaceMemory();
}

void Net::AppendTop(const NetParameter& param, const int layer_id, const int top_id,
                    std::set<string>* available_blobs, std::map<string, int>* blob_name_to_idx) {
  const LayerParameter& layer_param = LayerAt(param, layer_id);
  const string blob_name = layer_param.get_string("top", "(automatic)", top_id);
  if (layer_param.count("bottom") > top_id &&
      blob_name == layer_param.get_string("bottom", "", top_id)) {
    // In-place: the top is the bottom's blob.
    const int blob_id = (*blob_name_to_idx)[blob_name];
    top_vecs_[layer_id].push_back(blobs_[blob_id].get());
    top_id_vecs_[layer_id].push_back(blob_id);
    blob_life_time_[blob_id] = std::max(blob_life_time_[blob_id], layer_id + 1);
  } else if (blob_name_to_idx->find(blob_name) != blob_name_to_idx->end()) {
    LOG(FATAL) << "Top blob '" << blob_name << "' produced by multiple sources.";
  } else {
    shared_ptr<Blob> blob_pointer(new Blob());
    const int blob_id = static_cast<int>(blobs_.size());
    blobs_.push_back(blob_pointer);
    blob_names_.push_back(blob_name);
    blob_life_time_.push_back(layer_id + 1);
    (*blob_name_to_idx)[blob_name] = blob_id;
    top_id_vecs_[layer_id].push_back(blob_id);
    top_vecs_[layer_id].push_back(blob_pointer.get());
  }
  available_blobs->insert(blob_name);
}

int Net::AppendBottom(const NetParameter& param, const int layer_id, const int bottom_id,
                      std::set<string>* available_blobs,
                      std::map<string, int>* blob_name_to_idx) {
  const LayerParameter& layer_param = LayerAt(param, layer_id);
  const string blob_name = layer_param.get_string("bottom", "", bottom_id);
  if (available_blobs->find(blob_name) == available_blobs->end()) {
    LOG(FATAL) << "Unknown bottom blob '" << blob_name << "' (layer '"
               << layer_param.get_string("name") << "', bottom index " << bottom_id << ")";
  }
  const int blob_id = (*blob_name_to_idx)[blob_name];
  bottom_vecs_[layer_id].push_back(blobs_[blob_id].get());
  bottom_id_vecs_[layer_id].push_back(blob_id);
  blob_life_time_[blob_id] = std::max(blob_life_time_[blob_id], layer_id);
  return blob_id;
}

void Net::AppendParam(const NetParameter& param, const int layer_id, const int param_id) {
  const LayerParameter& layer_param = layers_[layer_id]->layer_param();
  string param_name;
  if (layer_param.count("param") > param_id)
    param_name = layer_param.sub("param", param_id).get_string("name");
  if (param_name.empty()) {
    std::ostringstream os;
    os << layer_param.get_string("name") << "_" << param_id;
    param_name = os.str();
  }
  param_display_names_.push_back(param_name);
  const int net_param_id = static_cast<int>(params_.size());
  params_.push_back(layers_[layer_id]->blobs()[param_id]);
  param_id_vecs_[layer_id].push_back(net_param_id);
}

// Greedy buffer sharing over blob lifetimes (reference src/net.cpp:147-210): a
// top or scratch blob takes over the memory of a blob that is already dead if
// that block is big enough and at most twice too big.  Because all device work
// of a net is ordered on one stream, a block can be handed on as soon as the
// layer that last read it has been queued.  Shapes rarely change between
// calls, so the placement is recomputed only when they did.
void Net::PlaceMemory() {
  this->Reshape();
  if (fusion_dirty_) {
    PlanFusion();  // decides which tops alias their producer's blob
    placed_shapes_.clear();
  }
  vector<vector<int> > shapes;
  shapes.reserve(blobs_.size());
  for (auto& b : blobs_) shapes.push_back(b->shape());
  vector<Blob*> all_temps;
  for (auto& l : layers_)
    for (Blob* t : l->GetTempBlobs()) {
      all_temps.push_back(t);
      shapes.push_back(t->shape());
    }
  if (shapes == placed_shapes_) return;
  placed_shapes_ = shapes;

  typedef std::pair<size_t, Blob*> BlobPair;
  std::multimap<size_t, Blob*> pool;
  // A blob that the top of a folded sum or of a view aliases lives on under that
  // top's name: it is handed back to the pool when the top dies, not when the
  // blob does.
  std::set<int> kept_alive;
  for (int id : residual_alias_)
    if (id >= 0) kept_alive.insert(id);
  for (size_t i = 0; i < layers_.size(); ++i) {
    vector<Blob*> temps = layers_[i]->GetTempBlobs();
    vector<Blob*>& bottoms = bottom_vecs_[i];
    vector<Blob*>& tops = top_vecs_[i];
    vector<BlobPair> to_place;
    if (residual_alias_[i] >= 0) {
      // folded sum or view: no scratch, and the top is the aliased blob under a new name
      temps.clear();
      tops[0]->ResetMemory();
      tops[0]->ShareData(*blobs_[residual_alias_[i]]);
    } else {
      for (Blob* blob : temps) {
        blob->ResetMemory();
        to_place.push_back(std::make_pair(static_cast<size_t>(blob->count()), blob));
      }
      if (sibling_owner_[i] < 0) {  // a merged sibling's top was placed with its owner's
        for (Blob* blob : tops) {
          if (std::find(bottoms.begin(), bottoms.end(), blob) != bottoms.end()) continue;  // in place
          blob->ResetMemory();
          to_place.push_back(std::make_pair(static_cast<size_t>(blob->count()), blob));
        }
      }
      for (size_t j = i + 1; j < layers_.size() && j <= i + 8; ++j) {
        if (sibling_owner_[j] != static_cast<int>(i)) continue;
        for (Blob* blob : top_vecs_[j]) {  // written by this layer's launch
          blob->ResetMemory();
          to_place.push_back(std::make_pair(static_cast<size_t>(blob->count()), blob));
        }
      }
    }
    std::sort(to_place.begin(), to_place.end(),
              [](const BlobPair& x, const BlobPair& y) { return x.first > y.first; });
    for (auto& p : to_place) {
      auto it = pool.lower_bound(p.first);
      if (it != pool.end() && it->first <= p.first * 2) {
        p.second->ShareData(*it->second);
        pool.erase(it);
      }
    }
    std::set<int> released;  // a blob listed twice as bottom is released once
    for (int blob_idx : bottom_id_vecs_[i]) {
      if (blob_life_time_[blob_idx] <= static_cast<int>(i) && !kept_alive.count(blob_idx) &&
          released.insert(blob_idx).second) {
        pool.insert(std::make_pair(static_cast<size_t>(blobs_[blob_idx]->capacity()),
                                   blobs_[blob_idx].get()));
      }
    }
    for (Blob* blob : temps)
      pool.insert(std::make_pair(static_cast<size_t>(blob->capacity()), blob));
  }
}

// Finds runs  contraction -> in-place per-channel stages [-> activation]  and
// hands the followers to the contraction layer.  A follower qualifies only if
// it directly follows in layer order and reads and writes the contraction's top
// blob in place, so skipping it leaves that blob exactly as the unfused chain
// would (the Caffe idiom Conv -> BatchNorm -> Scale -> ReLU).
void Net::PlanFusion() {
  fusion_dirty_ = false;
  layer_fused_.assign(layers_.size(), 0);
  sibling_owner_.assign(layers_.size(), -1);
  for (auto& l : layers_) l->AdoptSibling(nullptr, nullptr);
  for (size_t i = 0; i < layers_.size(); ++i) {
    if (layer_fused_[i] || !layers_[i]->AcceptsEpilogue()) continue;
    vector<Layer*> followers;
    if (top_vecs_[i].size() == 1 && top_vecs_[i][0]->num_axes() >= 2) {
      Blob* t = top_vecs_[i][0];
      const int channels = t->shape(1);
      size_t j = i + 1;
      int affine = 0;
      while (j < layers_.size() && bottom_vecs_[j].size() == 1 && top_vecs_[j].size() == 1 &&
             bottom_vecs_[j][0] == t && top_vecs_[j][0] == t &&
             layers_[j]->IsChannelStage(channels)) {
        const string ty = layers_[j]->type();
        const bool is_act = ty == "ReLU" || ty == "TanH" || ty == "Sigmoid";
        if (!layers_[i]->AcceptsFollower(layers_[j].get())) break;
        if (!is_act && ++affine > layers_[i]->MaxAffineFollowers()) break;
        followers.push_back(layers_[j].get());
        ++j;
        if (is_act) break;  // an activation ends the run
      }
    }
    layers_[i]->SetEpilogue(followers);
    for (size_t k = 0; k < followers.size(); ++k) layer_fused_[i + 1 + k] = 1;
  }

  // Residual sums (ResNet's  Eltwise(shortcut, branch) -> ReLU): when one input
  // of a two-input unit-coefficient sum comes straight from a contraction that
  // nothing else reads, and the other input is complete before that
  // contraction runs, the contraction adds it (and applies the sum's
  // activation) in its epilogue; the sum's top then aliases the contraction's
  // top blob and the sum itself is skipped.
  residual_alias_.assign(layers_.size(), -1);
  for (size_t e = 0; e < layers_.size(); ++e) {
    if (layer_fused_[e] || !layers_[e]->IsPlainSum()) continue;
    if (bottom_vecs_[e].size() != 2 || top_vecs_[e].size() != 1) continue;
    Blob* E = top_vecs_[e][0];
    if (E == bottom_vecs_[e][0] || E == bottom_vecs_[e][1]) continue;
    if (bottom_vecs_[e][0] == bottom_vecs_[e][1]) continue;
    auto last_writer = [&](const Blob* b, int before) {
      for (int j = before - 1; j >= 0; --j)
        if (std::find(top_vecs_[j].begin(), top_vecs_[j].end(), b) != top_vecs_[j].end()) return j;
      return -1;
    };
    // the input written last is the candidate; the other one is the residual
    const int w0 = last_writer(bottom_vecs_[e][0], static_cast<int>(e));
    const int w1 = last_writer(bottom_vecs_[e][1], static_cast<int>(e));
    const int ti = w0 > w1 ? 0 : 1;
    Blob* T = bottom_vecs_[e][ti];
    Blob* R = bottom_vecs_[e][1 - ti];
    const int t_id = bottom_id_vecs_[e][ti];
    int c = std::max(w0, w1);
    const int r_writer = std::min(w0, w1);
    while (c >= 0 && layer_fused_[c]) --c;  // walk back over the folded in-place stages
    if (c < 0 || r_writer >= c) continue;
    if (!layers_[c]->AcceptsEpilogue() || !layers_[c]->AcceptsResidual()) continue;
    if (top_vecs_[c].size() != 1 || top_vecs_[c][0] != T) continue;
    if (blob_life_time_[t_id] != static_cast<int>(e)) continue;  // read later, or an output
    bool exclusive = true;
    for (size_t j = c + 1; j < e && exclusive; ++j) {
      if (layer_fused_[j]) continue;
      for (Blob* b : bottom_vecs_[j])
        if (b == T) exclusive = false;
      for (Blob* b : top_vecs_[j])
        if (b == T || b == R) exclusive = false;
    }
    if (!exclusive || T->shape() != R->shape()) continue;
    layers_[c]->SetResidual(R, layers_[e]->AbsorbedActivation());
    layer_fused_[e] = 1;
    residual_alias_[e] = t_id;
  }

  // Sibling convolutions (the loc and conf heads of an SSD source): two layers
  // with one bottom and one top each that read the same blob with the same
  // window geometry and have nothing folded in run as one launch of the first.
  // The second's top must not exist before the second layer, and nothing between
  // the two may write the shared bottom.
  for (size_t i = 0; i < layers_.size(); ++i) {
    vector<int> key_i, key_j;
    if (layer_fused_[i] || bottom_vecs_[i].size() != 1 || top_vecs_[i].size() != 1) continue;
    if (bottom_vecs_[i][0] == top_vecs_[i][0] || !layers_[i]->SiblingKey(&key_i)) continue;
    Blob* shared = bottom_vecs_[i][0];
    for (size_t j = i + 1; j < layers_.size() && j <= i + 8; ++j) {
      bool writes_shared = false;
      for (Blob* b : top_vecs_[j]) writes_shared = writes_shared || b == shared;
      if (writes_shared) break;
      if (layer_fused_[j] || sibling_owner_[j] >= 0) continue;
      if (bottom_vecs_[j].size() != 1 || top_vecs_[j].size() != 1 || bottom_vecs_[j][0] != shared) continue;
      Blob* top_j = top_vecs_[j][0];
      if (top_j == shared || top_j == top_vecs_[i][0]) continue;
      if (std::string(layers_[j]->type()) != layers_[i]->type()) continue;
      if (!layers_[j]->SiblingKey(&key_j) || key_i != key_j) continue;
      bool seen_before = false;
      for (size_t k = 0; k < j && !seen_before; ++k) {
        for (Blob* b : top_vecs_[k]) seen_before = seen_before || b == top_j;
        for (Blob* b : bottom_vecs_[k]) seen_before = seen_before || b == top_j;
      }
      if (seen_before) continue;
      layers_[i]->AdoptSibling(layers_[j].get(), top_j);
      layer_fused_[j] = 1;
      sibling_owner_[j] = static_cast<int>(i);
      break;  // one sibling per layer
    }
  }

  // Views (Flatten, Reshape; the reference copies, src/layers/flatten_layer.cpp:34-39,
  // reshape_layer.cpp:98-103): when the view is the last reader of its bottom and
  // the bottom is neither a net input nor a marked output, the top takes over the
  // bottom's memory and the copy is skipped.
  for (size_t v = 0; v < layers_.size(); ++v) {
    if (layer_fused_[v] || !layers_[v]->IsView()) continue;
    if (bottom_vecs_[v].size() != 1 || top_vecs_[v].size() != 1) continue;
    if (bottom_vecs_[v][0] == top_vecs_[v][0]) continue;
    const int b_id = bottom_id_vecs_[v][0];
    if (blob_life_time_[b_id] != static_cast<int>(v)) continue;
    // a bottom that its producer re-shapes (and may re-allocate) in Forward
    // cannot be aliased ahead of time: the view copies instead
    bool late_shape = false;
    for (size_t w = 0; w < v; ++w)
      if (layers_[w]->ShapesTopInForward() &&
          std::find(top_vecs_[w].begin(), top_vecs_[w].end(), bottom_vecs_[v][0]) != top_vecs_[w].end())
        late_shape = true;
    if (late_shape) continue;
    layer_fused_[v] = 1;
    residual_alias_[v] = b_id;
  }
}

void Net::Forward(bool reshape) {
  CHECK(Context::mode() == GPU)
      << "Net::Forward: this library implements the HIP device path only; call "
      << "SetMode(GPU, device) on this thread first";
  if (reshape || fusion_dirty_) PlaceMemory();
  Profiler* profiler = Profiler::Get();
  const bool profiling = profiler->enabled();
  for (size_t i = 0; i < layers_.size(); ++i) {
    if (layer_fused_[i]) continue;
    if (profiling) profiler->ScopeStart(layer_names_[i].c_str());
    layers_[i]->Forward(bottom_vecs_[i], top_vecs_[i]);
    if (profiling) {
      Context::Get().Sync();  // scopes must cover device time
      profiler->ScopeEnd();
    }
  }
  // Bring the outputs of the last layer back, as the reference does
  // (src/net.cpp:226-232); this is also the one stream synchronisation of the pass.
  if (profiling) profiler->ScopeStart("Sync");
  for (Blob* blob : top_vecs_[layers_.size() - 1]) blob->cpu_data();
  Context::Get().Sync();
  if (profiling) profiler->ScopeEnd();
}

void Net::Reshape() {
  for (size_t i = 0; i < layers_.size(); ++i) layers_[i]->Reshape(bottom_vecs_[i], top_vecs_[i]);
}

void Net::CopyTrainedLayersFrom(const NetParameter& param) {
  // Accept both current `layer` and V1 `layers` entries: only name and blobs matter.
  for (const char* field : {"layer", "layers"}) {
    const int n = param.count(field);
    for (int i = 0; i < n; ++i) {
      const Message& source_layer = param.sub(field, i);
      const string source_layer_name = source_layer.get_string("name");
      auto it = layer_names_index_.find(source_layer_name);
      if (it == layer_names_index_.end()) continue;
      vector<shared_ptr<Blob> >& target_blobs = layers_[it->second]->blobs();
      CHECK_EQ(static_cast<int>(target_blobs.size()), source_layer.count("blobs"))
          << "Incompatible number of blobs for layer " << source_layer_name;
      for (size_t j = 0; j < target_blobs.size(); ++j) {
        const BlobProto& src =
            static_cast<const BlobProto&>(source_layer.sub("blobs", static_cast<int>(j)));
        if (!target_blobs[j]->ShapeEquals(src)) {
          Blob source_blob;
          source_blob.FromProto(src, true);
          LOG(FATAL) << "Cannot copy param " << j << " weights from layer '" << source_layer_name
                     << "'; shape mismatch.  Source param shape is " << source_blob.shape_string()
                     << "; target param shape is " << target_blobs[j]->shape_string() << ". "
                     << "To learn this layer's parameters from scratch rather than "
                     << "copying from a saved net, rename the layer.";
        }
        target_blobs[j]->FromProto(src, false);
      }
    }
  }
}

void Net::CopyTrainedLayersFrom(const string& trained_filename) {
  NetParameter param;
  ReadNetParamsFromBinaryFileOrDie(trained_filename, &param);
  CopyTrainedLayersFrom(param);
}

void Net::MarkOutputs(const std::vector<std::string>& outs) {
  for (const auto& name : outs) {
    auto it = blob_names_index_.find(name);
    if (it == blob_names_index_.end()) LOG(FATAL) << "blob (" << name << ") is not availiable in Net";
    blob_life_time_[it->second] = static_cast<int>(layers_.size());
  }
  placed_shapes_.clear();  // lifetimes changed: place again on the next Forward
  fusion_dirty_ = true;    // and a blob that is now an output must keep its own values
}

const vector<int>& Net::top_ids(int i) const {
  CHECK_GE(i, 0) << "Invalid layer id";
  CHECK_LT(i, static_cast<int>(top_id_vecs_.size())) << "Invalid layer id";
  return top_id_vecs_[i];
}

const vector<int>& Net::bottom_ids(int i) const {
  CHECK_GE(i, 0) << "Invalid layer id";
  CHECK_LT(i, static_cast<int>(bottom_id_vecs_.size())) << "Invalid layer id";
  return bottom_id_vecs_[i];
}

bool Net::has_blob(const string& blob_name) const {
  return blob_names_index_.find(blob_name) != blob_names_index_.end();
}

const shared_ptr<Blob> Net::blob_by_name(const string& blob_name) const {
  CHECK(has_blob(blob_name)) << "Unknown blob name " << blob_name;
  return blobs_[blob_names_index_.find(blob_name)->second];
}

// reference src/net.cpp:293-301
void Net::ToProto(NetParameter* param) const {
  param->fields().clear();
  param->set("name", name_, true);
  for (const auto& layer : layers_)
    layer->ToProto(static_cast<LayerParameter*>(param->add_sub("layer")));
}

shared_ptr<NetParameter> ReadTextNetParameterFromFile(const string& file) {
  shared_ptr<NetParameter> np(new NetParameter);
  ReadNetParamsFromTextFileOrDie(file, np.get());
  return np;
}

shared_ptr<NetParameter> ReadTextNetParameterFromBuffer(const char* buffer, int buffer_len) {
  shared_ptr<NetParameter> np(new NetParameter);
  ParseText(buffer, static_cast<size_t>(buffer_len), np.get());
  UpgradeNetAsNeeded("(buffer)", np.get());
  return np;
}

shared_ptr<NetParameter> ReadBinaryNetParameterFromFile(const string& file) {
  shared_ptr<NetParameter> np(new NetParameter);
  ReadNetParamsFromBinaryFileOrDie(file, np.get());
  return np;
}

shared_ptr<NetParameter> ReadBinaryNetParameterFromBuffer(const char* buffer, int buffer_len) {
  shared_ptr<NetParameter> np(new NetParameter);
  ParseBinaryNet(reinterpret_cast<const uint8_t*>(buffer), static_cast<size_t>(buffer_len),
                 np.get());
  return np;
}

}  // namespace caffe
