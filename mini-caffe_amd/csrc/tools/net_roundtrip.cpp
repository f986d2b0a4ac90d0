// Re-serialises a net and checks that nothing is lost:
//
//   net_roundtrip net.prototxt weights.caffemodel out.caffemodel
//
// 1. builds the net and copies the trained blobs in;
// 2. Net::ToProto -> a second Net built from that NetParameter alone (the layer
//    constructors take their blobs from the definition): every parameter blob must
//    equal the first net's bit for bit;
// 3. the same NetParameter through the library's wire-format writer and reader into
//    a third net: equal again.  The bytes are also written to out.caffemodel so that
//    a caller can walk them with a reader of its own.
// Runs without a device (no Forward).  Exit code 0 and a line "roundtrip ok: N
// parameter blobs" on success.
#include <cstdio>
#include <cstring>
#include <fstream>
#include <string>

#include <caffe/net.hpp>

#include "proto.hpp"

namespace {

int compare(const caffe::Net& a, const caffe::Net& b, const char* what) {
  CHECK_EQ(a.params().size(), b.params().size()) << what;
  CHECK(a.param_names() == b.param_names()) << what << ": parameter names differ";
  for (size_t i = 0; i < a.params().size(); ++i) {
    const caffe::Blob& x = *a.params()[i];
    const caffe::Blob& y = *b.params()[i];
    CHECK(x.shape() == y.shape()) << what << ": shape of " << a.param_names()[i];
    CHECK_EQ(0, std::memcmp(x.cpu_data(), y.cpu_data(), sizeof(float) * x.count()))
        << what << ": values of " << a.param_names()[i];
  }
  return static_cast<int>(a.params().size());
}

}  // namespace

int main(int argc, char* argv[]) {
  CHECK_EQ(argc, 4) << "[Usage]: ./net_roundtrip net.prototxt weights.caffemodel out.caffemodel";
  try {
    caffe::Net first(argv[1]);
    first.CopyTrainedLayersFrom(std::string(argv[2]));

    std::shared_ptr<caffe::NetParameter> param = caffe::ReadTextNetParameterFromBuffer("", 0);
    first.ToProto(param.get());
    caffe::Net second(*param);
    CHECK(second.name() == first.name());
    CHECK(second.layer_names() == first.layer_names());
    CHECK(second.blob_names() == first.blob_names());
    const int n = compare(first, second, "ToProto -> Net");

    const std::string bytes = caffe::SerializeBinaryNet(*param);
    std::ofstream(argv[3], std::ios::binary).write(bytes.data(), bytes.size());
    std::shared_ptr<caffe::NetParameter> back =
        caffe::ReadBinaryNetParameterFromBuffer(bytes.data(), static_cast<int>(bytes.size()));
    caffe::Net third(argv[1]);
    third.CopyTrainedLayersFrom(*back);
    compare(first, third, "ToProto -> wire format -> CopyTrainedLayersFrom");
    std::printf("roundtrip ok: %d parameter blobs, %zu bytes\n", n, bytes.size());
  } catch (const caffe::Error& e) {
    std::fprintf(stderr, "net_roundtrip: %s\n", e.what());
    return 1;
  }
  return 0;
}
