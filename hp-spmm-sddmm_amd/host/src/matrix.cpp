#include "starml/matrix.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "hpspmm.h"

extern "C" {
void hpspmm_gen_dense_normal(uint64_t seed, int64_t count, float* out);
void hpspmm_gen_dense_uniform(uint64_t seed, int64_t count, float lo, float hi, float* out);
}

namespace starml {

namespace {

uint64_t g_seed = 0;
uint64_t g_draws = 0;  // every rand()/randn() call takes a fresh stream

void hip_check(hipError_t e, const char* what) {
  if (e != hipSuccess) throw Error(std::string(what) + ": " + hipGetErrorString(e));
}

std::shared_ptr<void> allocate(const Device& dev, size_t bytes) {
  if (bytes == 0) bytes = 1;
  if (dev.is_cpu()) {
    void* p = std::malloc(bytes);
    if (!p) throw Error("host allocation failed");
    return std::shared_ptr<void>(p, [](void* q) { std::free(q); });
  }
  if (dev.is_hip()) {
    hip_check(hipSetDevice(dev.index()), "hipSetDevice");
    void* p = nullptr;
    hip_check(hipMalloc(&p, bytes), "hipMalloc");
    return std::shared_ptr<void>(p, [](void* q) { (void)hipFree(q); });
  }
  throw Error("Matrix: device type not set");
}

}  // namespace

size_t DataType::size() const {
  switch (kind_) {
    case kInt32: return 4;
    case kInt64: return 8;
    case kFloat: return 4;
    case kDouble: return 8;
    default: throw Error("DataType: kind not set");
  }
}

Matrix::Matrix(const Shape& shape, const Device& device, const DataType& data_type)
    : device_(device), dtype_(data_type), shape_(shape) {
  size_ = 1;
  for (int64_t d : shape_) {
    if (d < 0) throw Error("Matrix: negative dimension");
    size_ *= d;
  }
  data_ = allocate(device_, (size_t)size_ * dtype_.size());
}

Matrix Matrix::to(Device new_device) const {
  Matrix out(shape_, new_device, dtype_);
  const size_t bytes = nbytes();
  if (bytes == 0) return out;
  if (device_.is_cpu() && new_device.is_cpu()) {
    std::memcpy(out.data_.get(), data_.get(), bytes);
    return out;
  }
  const hipMemcpyKind kind = device_.is_cpu() ? hipMemcpyHostToDevice
                             : new_device.is_cpu() ? hipMemcpyDeviceToHost
                                                   : hipMemcpyDeviceToDevice;
  hip_check(hipMemcpy(out.data_.get(), data_.get(), bytes, kind), "hipMemcpy");
  return out;
}

Matrix empty(const Shape& shape, const Device& device, const DataType& data_type) {
  return Matrix(shape, device, data_type);
}

Matrix full(const Shape& shape, const Device& device, const DataType& data_type, double init_val) {
  // FP32 on the device: allocated there and filled by a kernel, as the reference does
  // (spmm/starml/operators/cuda/factories_kernel.cu:8-17) - nothing crosses PCIe
  if (device.is_hip() && data_type.type() == kFloat) {
    Matrix out(shape, device, data_type);
    if (hpspmm_fill_f32(out.mutable_data<float>(), out.size(), (float)init_val, nullptr) != HPSPMM_OK)
      throw Error(std::string("full: ") + hpspmm_last_error());
    hip_check(hipStreamSynchronize(nullptr), "full");
    return out;
  }
  // other types (index arrays, host matrices): filled on the host, then moved
  Matrix host(shape, Device(kCPU), data_type);
  const int64_t n = host.size();
  switch (data_type.type()) {
    case kInt32: std::fill_n(host.mutable_data<int32_t>(), n, (int32_t)init_val); break;
    case kInt64: std::fill_n(host.mutable_data<int64_t>(), n, (int64_t)init_val); break;
    case kFloat: std::fill_n(host.mutable_data<float>(), n, (float)init_val); break;
    case kDouble: std::fill_n(host.mutable_data<double>(), n, init_val); break;
    default: throw Error("full: unsupported data type");
  }
  return device.is_cpu() ? host : host.to(device);
}

void set_rand_seed(uint64_t seed) {
  g_seed = seed;
  g_draws = 0;
}

Matrix rand(const Shape& shape, const Device& device, const DataType& data_type, double start, double end) {
  if (data_type.type() != kFloat) throw Error("rand: only float is supported");
  Matrix host(shape, Device(kCPU), data_type);
  hpspmm_gen_dense_uniform(g_seed + 7919 * (g_draws++), host.size(), (float)start, (float)end,
                           host.mutable_data<float>());
  return device.is_cpu() ? host : host.to(device);
}

Matrix randn(const Shape& shape, const Device& device, const DataType& data_type) {
  if (data_type.type() != kFloat) throw Error("randn: only float is supported");
  Matrix host(shape, Device(kCPU), data_type);
  hpspmm_gen_dense_normal(g_seed + 7919 * (g_draws++), host.size(), host.mutable_data<float>());
  return device.is_cpu() ? host : host.to(device);
}

}  // namespace starml
