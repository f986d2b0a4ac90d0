/*
 * Blob: an N-d float array mirrored lazily between host and HIP device memory.
 * Public surface of reference include/caffe/blob.hpp:25-266 (shape queries,
 * cpu/gpu data accessors, ShareData, FromProto/ToProto) over this build's
 * SyncedMemory.  Layout is contiguous row-major; for 4 axes that is NCHW with
 * offset ((n*C + c)*H + h)*W + w.
 */
#ifndef CAFFE_BLOB_HPP_
#define CAFFE_BLOB_HPP_

#include <string>
#include <vector>

#include "caffe/base.hpp"

namespace caffe {

class SyncedMemory;
class BlobProto;

const int kMaxBlobAxes = 32;

class CAFFE_API Blob {
 public:
  Blob() : count_(0), capacity_(0), own_data_(true) {}
  explicit Blob(const int num, const int channels, const int height, const int width);
  explicit Blob(const vector<int>& shape);

  void Reshape(const int num, const int channels, const int height, const int width);
  /*! \brief change the dimensions; memory is (re)allocated lazily and only grows */
  void Reshape(const vector<int>& shape);
  void ReshapeLike(const Blob& other) { Reshape(other.shape()); }

  string shape_string() const;
  const vector<int>& shape() const { return shape_; }
  int shape(int index) const { return shape_[CanonicalAxisIndex(index)]; }
  int num_axes() const { return static_cast<int>(shape_.size()); }
  int count() const { return count_; }
  int capacity() const { return capacity_; }
  /*! \brief product of extents of axes [start_axis, end_axis) */
  int count(int start_axis, int end_axis) const;
  int count(int start_axis) const { return count(start_axis, num_axes()); }
  /*! \brief map a possibly negative axis index into [0, num_axes) */
  int CanonicalAxisIndex(int axis_index) const;

  int num() const { return LegacyShape(0); }
  int channels() const { return LegacyShape(1); }
  int height() const { return LegacyShape(2); }
  int width() const { return LegacyShape(3); }
  int LegacyShape(int index) const;

  int offset(const int n, const int c = 0, const int h = 0, const int w = 0) const;
  int offset(const vector<int>& indices) const;

  real_t data_at(const int n, const int c, const int h, const int w) const {
    return cpu_data()[offset(n, c, h, w)];
  }
  real_t data_at(const vector<int>& index) const { return cpu_data()[offset(index)]; }

  const shared_ptr<SyncedMemory>& data() const { return data_; }

  const real_t* cpu_data() const;
  real_t* mutable_cpu_data();
  const real_t* gpu_data() const;
  real_t* mutable_gpu_data();
  /*! \brief the shape as a device int array (for kernels that take it by pointer) */
  const int* gpu_shape() const;

  void FromProto(const BlobProto& proto, bool reshape = true);
  void ToProto(BlobProto* proto) const;
  bool ShapeEquals(const BlobProto& other);

  /*! \brief alias another blob's memory; counts need not match, capacity must suffice */
  void ShareData(const Blob& other);
  /*! \brief stop aliasing another blob: take a fresh block of this blob's capacity */
  void ResetMemory();

  const string& name() const { return name_; }
  void set_name(const string& name) { name_ = name; }

 protected:
  shared_ptr<SyncedMemory> data_;
  mutable shared_ptr<SyncedMemory> shape_data_;
  vector<int> shape_;
  int count_;
  int capacity_;
  bool own_data_;
  string name_;

  DISABLE_COPY_AND_ASSIGN(Blob);
};

/*! \brief a Blob whose storage is read as 32-bit ints (reference blob.hpp BlobInt) */
class CAFFE_API BlobInt : public Blob {
 public:
  BlobInt() : Blob() {}
  const int* cpu_data() const { return reinterpret_cast<const int*>(Blob::cpu_data()); }
  int* mutable_cpu_data() { return reinterpret_cast<int*>(Blob::mutable_cpu_data()); }
  const int* gpu_data() const { return reinterpret_cast<const int*>(Blob::gpu_data()); }
  int* mutable_gpu_data() { return reinterpret_cast<int*>(Blob::mutable_gpu_data()); }
};

}  // namespace caffe

#endif  // CAFFE_BLOB_HPP_
