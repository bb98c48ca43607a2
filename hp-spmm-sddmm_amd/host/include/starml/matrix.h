// Dense buffer type of the host layer: shape + device + dtype + shared ownership.
//
// It keeps the surface the reference's SpMM drivers use from starml::Matrix
// (include/starml/basic/matrix.h:14-77: size(), dim(), dims(), ndims(),
// data<T>(), mutable_data<T>(), to(device), shallow copies sharing one
// allocation) with a HIP device backend and 64-bit sizes (the reference keeps
// element counts and byte counts in int, matrix.h:71, copy_kernel.cu:12).
// Only what the SpMM path touches is here: no broadcasting arithmetic, no
// dispatcher registry, no logger.
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace starml {

enum class DeviceType : int { UNCERTAIN = -1, CPU = 0, HIP = 1 };
constexpr DeviceType kCPU = DeviceType::CPU;
constexpr DeviceType kHIP = DeviceType::HIP;
// The reference spells the accelerator kCUDA (include/starml/basic/device.h:16);
// callers written against it keep compiling.
constexpr DeviceType kCUDA = DeviceType::HIP;

class Device {
 public:
  Device(DeviceType type = DeviceType::UNCERTAIN, int index = 0) : type_(type), index_(index) {}
  DeviceType type() const { return type_; }
  int index() const { return index_; }
  bool is_cpu() const { return type_ == kCPU; }
  bool is_hip() const { return type_ == kHIP; }
  bool is_cuda() const { return is_hip(); }
  bool operator==(const Device& o) const { return type_ == o.type_ && index_ == o.index_; }
  bool operator!=(const Device& o) const { return !(*this == o); }

 private:
  DeviceType type_;
  int index_;
};

enum class DataTypeKind : int { UNCERTAIN = -1, Int32 = 2, Int64 = 3, Float = 4, Double = 5 };
constexpr DataTypeKind kInt32 = DataTypeKind::Int32;
constexpr DataTypeKind kInt64 = DataTypeKind::Int64;
constexpr DataTypeKind kFloat = DataTypeKind::Float;
constexpr DataTypeKind kDouble = DataTypeKind::Double;

class DataType {
 public:
  DataType(DataTypeKind kind = DataTypeKind::UNCERTAIN) : kind_(kind) {}
  DataTypeKind type() const { return kind_; }
  size_t size() const;
  template <typename T>
  bool is_valid() const;
  bool operator==(const DataType& o) const { return kind_ == o.kind_; }

 private:
  DataTypeKind kind_;
};

template <> inline bool DataType::is_valid<int32_t>() const { return kind_ == kInt32; }
template <> inline bool DataType::is_valid<int64_t>() const { return kind_ == kInt64; }
template <> inline bool DataType::is_valid<float>() const { return kind_ == kFloat; }
template <> inline bool DataType::is_valid<double>() const { return kind_ == kDouble; }

using Shape = std::vector<int64_t>;

// Raised where the reference aborts through its check macros
// (include/starml/utils/loguru.h:1535-1542): wrong dtype in data<T>(), failed
// allocation or copy, malformed input file.
struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};

class Matrix {
 public:
  Matrix() = default;
  Matrix(const Shape& shape, const Device& device, const DataType& data_type);
  Matrix(const Shape& shape, const DataType& data_type, const Device& device)
      : Matrix(shape, device, data_type) {}

  int64_t size() const { return size_; }
  const Shape& dims() const { return shape_; }
  int64_t dim(int axis) const { return shape_.at((size_t)axis); }
  int ndims() const { return (int)shape_.size(); }
  const Device& device() const { return device_; }
  const DataType& data_type() const { return dtype_; }
  bool is_cuda() const { return device_.is_hip(); }
  size_t nbytes() const { return (size_t)size_ * dtype_.size(); }

  const void* raw_data() const { return data_.get(); }
  void* raw_mutable_data() const { return data_.get(); }

  template <typename T>
  const T* data() const {
    check_type(dtype_.is_valid<T>());
    return static_cast<const T*>(data_.get());
  }
  template <typename T>
  T* mutable_data() const {
    check_type(dtype_.is_valid<T>());
    return static_cast<T*>(data_.get());
  }

  // Deep copy onto another device (host<->device, device->device, host->host).
  // Synchronous, size_t byte counts.
  Matrix to(Device new_device) const;

 private:
  static void check_type(bool ok) {
    if (!ok) throw Error("Matrix::data<T>(): T does not match the matrix data type");
  }
  int64_t size_ = 0;
  Device device_;
  DataType dtype_;
  std::shared_ptr<void> data_;
  Shape shape_;
};

// Factories the SpMM drivers use (include/starml/operators/factories.h:12-17).
Matrix empty(const Shape& shape, const Device& device, const DataType& data_type);
Matrix full(const Shape& shape, const Device& device, const DataType& data_type, double init_val);
// U(start, end).  The reference seeds from std::random_device
// (spmm/starml/operators/cpu/factories_kernel.cpp:21-22) and is not
// reproducible; here the stream is seeded (set_rand_seed, default 0).
Matrix rand(const Shape& shape, const Device& device, const DataType& data_type, double start, double end);
// N(0, 1): the dense operand of the benchmark configurations.
Matrix randn(const Shape& shape, const Device& device, const DataType& data_type);
void set_rand_seed(uint64_t seed);

}  // namespace starml
