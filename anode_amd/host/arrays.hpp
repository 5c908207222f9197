// Device arrays and the connection handle as anode's host code describes them (src/ops_gpu.rs:670-679, the
// GPUDeviceOuterBatchArray{1,3,4}d family): packed, first-index-fastest arrays given by a device pointer and a Shape
// (`size` = the non-batch dimensions, fastest first, plus a batch size), and what a caller takes from its
// connection, conn.cuda_stream() and conn.cuda_kernel_config().  Shared by the staging layer (io_gpu.hpp) and by
// the test harness's mirror of the caller layer.
#pragma once

#define ANODE_DEFINE_KERNEL_CONFIG
#include "../../include/anode_routines_gpu.h"

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>

namespace anode_host {

// src/lib.rs:1810-1813
enum class WriteCap { Assign, Accumulate };

// the reference's `unimplemented!()`
struct Unimplemented : std::logic_error {
  explicit Unimplemented(const std::string &what) : std::logic_error("unimplemented: " + what) {}
};

// src/ops_gpu.rs:57-61: sizes must fit the ABI's u32
inline uint32_t sz2uint(size_t sz) {
  if (sz > 0xffffffffull) throw std::overflow_error("sz2uint: size does not fit in u32");
  return uint32_t(sz);
}

// What the Rust callers take from their connection: conn.cuda_stream() and
// conn.cuda_kernel_config() (src/ops_gpu.rs:670-679).
struct GPUDeviceConn {
  hipStream_t stream = nullptr;
  KernelConfig cfg{1024, 1024};
  const KernelConfig *cuda_kernel_config() const { return &cfg; }
  CUstream_st *cuda_stream() const { return reinterpret_cast<CUstream_st *>(stream); }
};

// Non-batch dimensions (fastest first) and the outer batch size.
struct Shape {
  size_t size[4] = {1, 1, 1, 1};
  int nd = 1;
  size_t batch = 1;
  size_t index_at(int i) const { return i < nd ? size[i] : batch; }  // the batch is the last axis
  size_t flat_len_upto(int n) const {                                // product of the first n axes
    size_t p = 1;
    for (int i = 0; i < n; ++i) p *= size[i];
    return p;
  }
  size_t flat_len() const { return flat_len_upto(nd) * batch; }
};

template <typename T>
struct DeviceArray {
  T *dptr = nullptr;
  Shape shape;
  bool packed = true;  // only packed arrays are implemented, as in the reference
  bool is_packed() const { return packed; }
  const T *as_dptr() const { return dptr; }
  T *as_mut_dptr() const { return dptr; }
};

inline DeviceArray<float> array1d(float *p, size_t n) {
  DeviceArray<float> a;
  a.dptr = p;
  a.shape.size[0] = n;
  a.shape.nd = 1;
  return a;
}

// [d0, batch]: GPUDeviceOuterBatchArray1d
template <typename T>
inline DeviceArray<T> obatch1d(T *p, size_t d0, size_t batch) {
  DeviceArray<T> a;
  a.dptr = p;
  a.shape.size[0] = d0;
  a.shape.nd = 1;
  a.shape.batch = batch;
  return a;
}

// [W, H, C, batch]: GPUDeviceOuterBatchArray3d (NCHW memory)
template <typename T>
inline DeviceArray<T> obatch3d(T *p, size_t w, size_t h, size_t c, size_t batch) {
  DeviceArray<T> a;
  a.dptr = p;
  a.shape.size[0] = w;
  a.shape.size[1] = h;
  a.shape.size[2] = c;
  a.shape.nd = 3;
  a.shape.batch = batch;
  return a;
}

// [X, Y, Z, C, batch]: GPUDeviceOuterBatchArray4d (NCDHW memory)
template <typename T>
inline DeviceArray<T> obatch4d(T *p, size_t x, size_t y, size_t z, size_t c, size_t batch) {
  DeviceArray<T> a;
  a.dptr = p;
  a.shape.size[0] = x;
  a.shape.size[1] = y;
  a.shape.size[2] = z;
  a.shape.size[3] = c;
  a.shape.nd = 4;
  a.shape.batch = batch;
  return a;
}

namespace detail {
// the reference's callers only implement packed arrays (src/ops_gpu.rs:3731-3779)
template <typename... A>
inline void require_packed(const char *op, const A &...arrays) {
  const bool packed = (arrays.is_packed() && ...);
  if (!packed) throw Unimplemented(std::string(op) + ": non-packed arrays");
}
}  // namespace detail

}  // namespace anode_host
