// Self-contained reader for the slice of caffe.proto that the forward path
// needs: protobuf text format (prototxt) and wire format (caffemodel).
//
// Stands in for the generated caffe.pb.{h,cc} + libprotobuf of the reference
// (reference src/proto/caffe.proto, src/util/io.cpp:34-72): there is no
// protobuf toolchain on the target.  Messages are kept as an ordered list of
// named fields, so layer code asks for "convolution_param" / "kernel_size" by
// name, for both sources alike.
#ifndef MCHIP_RUNTIME_PROTO_HPP_
#define MCHIP_RUNTIME_PROTO_HPP_

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "caffe/base.hpp"

namespace caffe {

class Message {
 public:
  struct Field {
    std::string name;
    std::string text;                 // scalar as written (number, identifier or string body)
    bool quoted = false;              // text came from a quoted string
    std::shared_ptr<Message> msg;     // nested message, if any
    std::shared_ptr<std::vector<float> > floats;  // bulk float payload (BlobProto.data)
  };

  int count(const std::string& name) const;
  bool has(const std::string& name) const { return count(name) > 0; }

  // Nested message `name` (idx-th occurrence); an empty message if absent, so
  // defaults apply the way protobuf's default instances do.
  const Message& sub(const std::string& name, int idx = 0) const;
  Message* add_sub(const std::string& name);

  long get_int(const std::string& name, long def = 0, int idx = 0) const;
  double get_float(const std::string& name, double def = 0., int idx = 0) const;
  bool get_bool(const std::string& name, bool def = false, int idx = 0) const;
  std::string get_string(const std::string& name, const std::string& def = "",
                         int idx = 0) const;

  void add(const std::string& name, const std::string& text, bool quoted = false);
  void add_int(const std::string& name, long v);
  void add_float(const std::string& name, double v);
  void set(const std::string& name, const std::string& text, bool quoted = false);
  void remove(const std::string& name);

  const Field* find(const std::string& name, int idx = 0) const;
  std::vector<Field>& fields() { return fields_; }
  const std::vector<Field>& fields() const { return fields_; }

  // Text-format rendering (round-trips through ParseText).
  std::string DebugString(int indent = 0) const;

 private:
  std::vector<Field> fields_;
};

// Named so that the public headers' forward declarations resolve.
class BlobProto : public Message {};
class LayerParameter : public Message {};
class NetParameter : public Message {};

// Protobuf text format -> Message.  Throws caffe::Error with line:column.
void ParseText(const char* data, size_t len, Message* out);
// Protobuf wire format of a NetParameter (a .caffemodel) -> Message.  Known
// fields are decoded by the schema in proto.cpp; unknown ones are skipped.
void ParseBinaryNet(const uint8_t* data, size_t len, Message* out);

void ReadNetParamsFromTextFileOrDie(const std::string& file, NetParameter* param);
void ReadNetParamsFromBinaryFileOrDie(const std::string& file, NetParameter* param);

// Rewrites V1 `layers { type: CONVOLUTION ... }` definitions as `layer` messages
// (reference src/util/upgrade_proto.cpp:60-265) and folds legacy top-level
// `input:` / `input_shape` / `input_dim` declarations into a leading Input layer
// (reference src/util/upgrade_proto.cpp:267-305).
void UpgradeNetAsNeeded(const std::string& source, NetParameter* param);

// Serialises a NetParameter holding name / layer{name,type,blobs} to wire format.
std::string SerializeBinaryNet(const Message& net);

}  // namespace caffe

#endif  // MCHIP_RUNTIME_PROTO_HPP_
