/*
 * Net: a DAG of layers built from a NetParameter (prototxt) and run forward.
 * Public surface of reference include/caffe/net.hpp:23-159.  In GPU mode the
 * forward pass runs on the calling thread's HIP stream; in-place
 * BatchNorm/Scale/Bias/activation followers of a contraction layer are folded
 * into that layer's kernel epilogue, which leaves every blob's final contents
 * as the unfused sequence would.
 */
#ifndef CAFFE_NET_HPP_
#define CAFFE_NET_HPP_

#include <map>
#include <set>
#include <string>
#include <utility>
#include <vector>

#include "caffe/blob.hpp"

namespace caffe {

class Layer;
class NetParameter;

class CAFFE_API Net {
 public:
  explicit Net(const string& param_file);
  explicit Net(const NetParameter& param) { Init(param); }
  ~Net();

  void Init(const NetParameter& param);

  /*!
   * \brief run all layers in order
   * \param reshape re-run every layer's Reshape first (needed after an input
   *        blob changed shape); buffers are re-placed only when shapes changed
   */
  void Forward(bool reshape = true);
  /*! \brief propagate shapes from the inputs through every layer */
  void Reshape();

  /*! \brief copy blobs of same-named layers from a trained net */
  void CopyTrainedLayersFrom(const NetParameter& param);
  void CopyTrainedLayersFrom(const string& trained_filename);

  /*! \brief the net's definition with every layer's current parameter blobs */
  void ToProto(NetParameter* param) const;

  const string& name() const { return name_; }
  const vector<string>& blob_names() const { return blob_names_; }
  const vector<string>& param_names() const { return param_display_names_; }
  const vector<string>& layer_names() const { return layer_names_; }
  const vector<shared_ptr<Blob> >& blobs() const { return blobs_; }
  const vector<shared_ptr<Blob> >& params() const { return params_; }
  const vector<shared_ptr<Layer> >& layers() const { return layers_; }
  const vector<vector<Blob*> >& bottom_vecs() const { return bottom_vecs_; }
  const vector<vector<Blob*> >& top_vecs() const { return top_vecs_; }
  const vector<vector<int> >& param_id_vecs() const { return param_id_vecs_; }
  const vector<int>& top_ids(int i) const;
  const vector<int>& bottom_ids(int i) const;
  bool has_blob(const string& blob_name) const;
  const shared_ptr<Blob> blob_by_name(const string& blob_name) const;

  /*! \brief keep these blobs alive to the end of Forward (their memory is not reused) */
  void MarkOutputs(const std::vector<std::string>& outs);

 protected:
  void AppendTop(const NetParameter& param, const int layer_id, const int top_id,
                 std::set<string>* available_blobs, std::map<string, int>* blob_name_to_idx);
  int AppendBottom(const NetParameter& param, const int layer_id, const int bottom_id,
                   std::set<string>* available_blobs, std::map<string, int>* blob_name_to_idx);
  void AppendParam(const NetParameter& param, const int layer_id, const int param_id);
  void PlaceMemory();
  void PlanFusion();

  string name_;
  vector<shared_ptr<Layer> > layers_;
  vector<string> layer_names_;
  std::map<string, int> layer_names_index_;
  vector<shared_ptr<Blob> > blobs_;
  vector<string> blob_names_;
  vector<int> blob_life_time_;
  std::map<string, int> blob_names_index_;
  vector<shared_ptr<Blob> > params_;
  vector<string> param_display_names_;
  vector<vector<int> > param_id_vecs_;
  vector<vector<Blob*> > bottom_vecs_;
  vector<vector<int> > bottom_id_vecs_;
  vector<vector<Blob*> > top_vecs_;
  vector<vector<int> > top_id_vecs_;
  // layers whose work was folded into an earlier layer's kernel
  vector<char> layer_fused_;
  // for a sum folded into the layer that produces one of its inputs, and for a
  // skipped view (Flatten, Reshape): the blob id whose memory the layer's top
  // aliases, else -1 (indexed by layer)
  vector<int> residual_alias_;
  // for a convolution that an earlier sibling computes together with its own
  // (same bottom, same window geometry): that sibling's layer id, else -1
  vector<int> sibling_owner_;
  // shapes of all blobs at the last PlaceMemory
  vector<vector<int> > placed_shapes_;
  bool fusion_dirty_ = true;
  DISABLE_COPY_AND_ASSIGN(Net);
};

CAFFE_API shared_ptr<NetParameter> ReadTextNetParameterFromFile(const string& file);
CAFFE_API shared_ptr<NetParameter> ReadTextNetParameterFromBuffer(const char* buffer,
                                                                  int buffer_len);
CAFFE_API shared_ptr<NetParameter> ReadBinaryNetParameterFromFile(const string& file);
CAFFE_API shared_ptr<NetParameter> ReadBinaryNetParameterFromBuffer(const char* buffer,
                                                                    int buffer_len);

}  // namespace caffe

#endif  // CAFFE_NET_HPP_
