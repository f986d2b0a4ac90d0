#include "caffe/blob.hpp"

#include <climits>
#include <cstring>
#include <sstream>

#include "device.hpp"
#include "proto.hpp"

namespace caffe {

Blob::Blob(const int num, const int channels, const int height, const int width)
    : count_(0), capacity_(0), own_data_(true) {
  Reshape(num, channels, height, width);
}

Blob::Blob(const vector<int>& shape) : count_(0), capacity_(0), own_data_(true) {
  Reshape(shape);
}

void Blob::Reshape(const int num, const int channels, const int height, const int width) {
  Reshape(vector<int>{num, channels, height, width});
}

void Blob::Reshape(const vector<int>& shape) {
  CHECK_LE(shape.size(), static_cast<size_t>(kMaxBlobAxes));
  long count = 1;
  for (size_t i = 0; i < shape.size(); ++i) {
    CHECK_GE(shape[i], 0) << "blob extent must be non-negative";
    count *= shape[i];
    CHECK_LE(count, static_cast<long>(INT_MAX)) << "blob size exceeds INT_MAX";
  }
  if (shape != shape_) shape_data_.reset();
  shape_ = shape;
  count_ = static_cast<int>(count);
  if (count_ > capacity_ || !data_) {
    capacity_ = count_;
    own_data_ = true;
    data_.reset(new SyncedMemory(static_cast<size_t>(capacity_) * sizeof(real_t)));
  }
}

string Blob::shape_string() const {
  std::ostringstream os;
  for (size_t i = 0; i < shape_.size(); ++i) os << shape_[i] << " ";
  os << "(" << count_ << ")";
  return os.str();
}

int Blob::count(int start_axis, int end_axis) const {
  CHECK_LE(start_axis, end_axis);
  CHECK_GE(start_axis, 0);
  CHECK_GE(end_axis, 0);
  CHECK_LE(start_axis, num_axes());
  CHECK_LE(end_axis, num_axes());
  int c = 1;
  for (int i = start_axis; i < end_axis; ++i) c *= shape_[i];
  return c;
}

int Blob::CanonicalAxisIndex(int axis_index) const {
  CHECK_GE(axis_index, -num_axes()) << "axis " << axis_index << " out of range for "
                                    << num_axes() << "-D Blob with shape " << shape_string();
  CHECK_LT(axis_index, num_axes()) << "axis " << axis_index << " out of range for "
                                   << num_axes() << "-D Blob with shape " << shape_string();
  return axis_index < 0 ? axis_index + num_axes() : axis_index;
}

int Blob::LegacyShape(int index) const {
  CHECK_LE(num_axes(), 4) << "Cannot use legacy accessors on Blobs with > 4 axes.";
  CHECK_LT(index, 4);
  CHECK_GE(index, -4);
  if (index >= num_axes() || index < -num_axes()) return 1;  // trailing axes of extent 1
  return shape(index);
}

int Blob::offset(const int n, const int c, const int h, const int w) const {
  CHECK_GE(n, 0);
  CHECK_LE(n, num());
  CHECK_GE(c, 0);
  CHECK_LE(c, channels());
  CHECK_GE(h, 0);
  CHECK_LE(h, height());
  CHECK_GE(w, 0);
  CHECK_LE(w, width());
  return ((n * channels() + c) * height() + h) * width() + w;
}

int Blob::offset(const vector<int>& indices) const {
  CHECK_LE(indices.size(), static_cast<size_t>(num_axes()));
  int off = 0;
  for (int i = 0; i < num_axes(); ++i) {
    off *= shape(i);
    if (static_cast<int>(indices.size()) > i) {
      CHECK_GE(indices[i], 0);
      CHECK_LT(indices[i], shape(i));
      off += indices[i];
    }
  }
  return off;
}

const real_t* Blob::cpu_data() const {
  CHECK(data_) << "blob '" << name_ << "' has no memory";
  return static_cast<const real_t*>(data_->cpu_data());
}
real_t* Blob::mutable_cpu_data() {
  CHECK(data_) << "blob '" << name_ << "' has no memory";
  return static_cast<real_t*>(data_->mutable_cpu_data());
}
const real_t* Blob::gpu_data() const {
  CHECK(data_) << "blob '" << name_ << "' has no memory";
  return static_cast<const real_t*>(data_->gpu_data());
}
real_t* Blob::mutable_gpu_data() {
  CHECK(data_) << "blob '" << name_ << "' has no memory";
  return static_cast<real_t*>(data_->mutable_gpu_data());
}

const int* Blob::gpu_shape() const {
  if (!shape_data_) {
    shape_data_.reset(new SyncedMemory(sizeof(int) * (shape_.empty() ? 1 : shape_.size())));
    int* p = static_cast<int*>(shape_data_->mutable_cpu_data());
    for (size_t i = 0; i < shape_.size(); ++i) p[i] = shape_[i];
  }
  return static_cast<const int*>(shape_data_->gpu_data());
}

void Blob::ShareData(const Blob& other) {
  CHECK_LE(count_, other.capacity_) << "ShareData: '" << other.name_ << "' is too small for '"
                                    << name_ << "'";
  CHECK(other.data_) << "ShareData: '" << other.name_ << "' has no memory";
  data_ = other.data_;
  capacity_ = other.capacity_;
  own_data_ = false;
}

void Blob::ResetMemory() {
  // Only a blob that aliases someone else's block needs a new one
  // (reference src/blob.cpp:104-109).
  if (!own_data_) {
    own_data_ = true;
    capacity_ = count_;
    data_.reset(new SyncedMemory(static_cast<size_t>(capacity_) * sizeof(real_t)));
  }
}

namespace {
// Shape carried by a BlobProto: `shape { dim }`, else the legacy 4 extents
// (reference src/blob.cpp:145-180).
vector<int> ProtoShape(const Message& proto) {
  vector<int> shape;
  if (proto.has("num") || proto.has("channels") || proto.has("height") || proto.has("width")) {
    shape = {static_cast<int>(proto.get_int("num", 1)), static_cast<int>(proto.get_int("channels", 1)),
             static_cast<int>(proto.get_int("height", 1)), static_cast<int>(proto.get_int("width", 1))};
  } else {
    const Message& s = proto.sub("shape");
    for (int i = 0; i < s.count("dim"); ++i) shape.push_back(static_cast<int>(s.get_int("dim", 0, i)));
  }
  return shape;
}
}  // namespace

bool Blob::ShapeEquals(const BlobProto& other) {
  const bool legacy = other.has("num") || other.has("channels") || other.has("height") ||
                      other.has("width");
  vector<int> s = ProtoShape(other);
  if (legacy) {
    // A legacy 4-D proto matches an N-d blob when the padded shapes agree
    // (reference src/blob.cpp:111-131).
    return num_axes() <= 4 && LegacyShape(-4) == s[0] && LegacyShape(-3) == s[1] &&
           LegacyShape(-2) == s[2] && LegacyShape(-1) == s[3];
  }
  return s == shape_;
}

void Blob::FromProto(const BlobProto& proto, bool reshape) {
  if (reshape) {
    Reshape(ProtoShape(proto));
  } else {
    CHECK(ShapeEquals(proto)) << "shape mismatch (reshape not set)";
  }
  real_t* dst = mutable_cpu_data();
  const Message::Field* bulk = nullptr;
  for (const auto& f : proto.fields())
    if (f.name == "data" && f.floats) bulk = &f;
  if (bulk) {
    CHECK_EQ(static_cast<int>(bulk->floats->size()), count_) << "blob data size mismatch";
    memcpy(dst, bulk->floats->data(), sizeof(real_t) * count_);
    return;
  }
  const char* field = proto.has("double_data") ? "double_data" : "data";
  const int n = proto.count(field);
  if (n == 0) return;  // shape only
  CHECK_EQ(n, count_) << "blob data size mismatch";
  int i = 0;
  for (const auto& f : proto.fields())
    if (f.name == field) dst[i++] = static_cast<real_t>(std::strtod(f.text.c_str(), nullptr));
}

void Blob::ToProto(BlobProto* proto) const {
  proto->fields().clear();
  Message* s = proto->add_sub("shape");
  for (int d : shape_) s->add_int("dim", d);
  Message::Field f;
  f.name = "data";
  f.floats = std::make_shared<std::vector<float> >(cpu_data(), cpu_data() + count_);
  proto->fields().push_back(f);
}

}  // namespace caffe
