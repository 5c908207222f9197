// Host <-> device staging either side of the operator path, in C++.
//
// The reference moves arrays with synchronous copies from and to pageable host
// memory (src/io_gpu.rs:286-330: `sync_copy_mem` on deserialize, `sync_dump_mem`
// on serialize) and then runs the cast / dequantize operator, or the host-side
// arg-max, as a separate step.  The first part of this file mirrors that pair.
//
// The second part is the MI355X-side input / output pipeline built on the same
// entry points:
//   * ImageBatchStager: u8 image batches travel from pinned host slots over a
//     dedicated copy stream while the previous batch is being converted; the
//     conversion is the one-pass dequantize + per-channel normalise
//     (anode_gpu_bcast_dequantize_u8_I1b_I2abc_Oabc_packed_f32), ordered after
//     the copy by an event, so the compute stream never waits on the host.
//   * LogitsArgMaxReader: the arg-max is taken on the device
//     (anode_gpu_arg_max_packed_u32, same tie / NaN rules as the host loop
//     src/utils/mod.rs:31-41) and only one u32 per row crosses to the host,
//     instead of the whole logits array.
//
// Streams are created at the default priority.  Pinned memory is allocated
// (hipHostMalloc), never registered.
#pragma once

#include "anode_amd/host/arrays.hpp"

#include <hip/hip_runtime.h>

#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace anode_host {

namespace detail {
inline void hip_ok(hipError_t e, const char *what) {
  if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}
}  // namespace detail

// ---------------------------------------------------------------------------
// the reference's pair (src/io_gpu.rs:286-330)
// ---------------------------------------------------------------------------

// deserialize: host -> device, complete on return
template <typename T>
inline void sync_copy_mem(DeviceArray<T> &dst, const T *host, const GPUDeviceConn &conn) {
  detail::require_packed("sync_copy_mem", dst);
  hipStream_t s = reinterpret_cast<hipStream_t>(conn.cuda_stream());
  detail::hip_ok(hipMemcpyAsync(dst.as_mut_dptr(), host, dst.shape.flat_len() * sizeof(T), hipMemcpyHostToDevice, s),
                 "sync_copy_mem");
  detail::hip_ok(hipStreamSynchronize(s), "sync_copy_mem");
}

// serialize: device -> host, complete on return
template <typename T>
inline void sync_dump_mem(const DeviceArray<T> &src, T *host, const GPUDeviceConn &conn) {
  detail::require_packed("sync_dump_mem", src);
  hipStream_t s = reinterpret_cast<hipStream_t>(conn.cuda_stream());
  detail::hip_ok(hipMemcpyAsync(host, src.as_dptr(), src.shape.flat_len() * sizeof(T), hipMemcpyDeviceToHost, s),
                 "sync_dump_mem");
  detail::hip_ok(hipStreamSynchronize(s), "sync_dump_mem");
}

// ---------------------------------------------------------------------------
// pinned host memory
// ---------------------------------------------------------------------------

template <typename T>
class PinnedBuffer {
 public:
  explicit PinnedBuffer(size_t count) : n_(count) {
    void *p = nullptr;
    detail::hip_ok(hipHostMalloc(&p, (count ? count : 1) * sizeof(T), hipHostMallocDefault), "hipHostMalloc");
    p_ = static_cast<T *>(p);
  }
  ~PinnedBuffer() { (void)hipHostFree(p_); }
  PinnedBuffer(const PinnedBuffer &) = delete;
  PinnedBuffer &operator=(const PinnedBuffer &) = delete;
  T *data() { return p_; }
  const T *data() const { return p_; }
  size_t size() const { return n_; }

 private:
  T *p_ = nullptr;
  size_t n_ = 0;
};

// Owning handles, so that a constructor that throws half-way leaks nothing.
template <typename T>
class DeviceBuffer {
 public:
  explicit DeviceBuffer(size_t count) {
    detail::hip_ok(hipMalloc(reinterpret_cast<void **>(&p_), (count ? count : 1) * sizeof(T)), "hipMalloc");
  }
  ~DeviceBuffer() { (void)hipFree(p_); }
  DeviceBuffer(const DeviceBuffer &) = delete;
  DeviceBuffer &operator=(const DeviceBuffer &) = delete;
  T *data() const { return p_; }

 private:
  T *p_ = nullptr;
};

class Event {
 public:
  Event() { detail::hip_ok(hipEventCreateWithFlags(&e_, hipEventDisableTiming), "hipEventCreate"); }
  ~Event() { (void)hipEventDestroy(e_); }
  Event(const Event &) = delete;
  Event &operator=(const Event &) = delete;
  hipEvent_t get() const { return e_; }

 private:
  hipEvent_t e_ = nullptr;
};

class CopyStream {  // default priority, does not synchronise with the null stream
 public:
  CopyStream() { detail::hip_ok(hipStreamCreateWithFlags(&s_, hipStreamNonBlocking), "hipStreamCreate"); }
  ~CopyStream() {
    (void)hipStreamSynchronize(s_);
    (void)hipStreamDestroy(s_);
  }
  CopyStream(const CopyStream &) = delete;
  CopyStream &operator=(const CopyStream &) = delete;
  hipStream_t get() const { return s_; }

 private:
  hipStream_t s_ = nullptr;
};

// ---------------------------------------------------------------------------
// u8 image batches in: copy stream + fused dequantize / normalise
// ---------------------------------------------------------------------------

// `depth` slots, each a pinned host buffer and a device u8 buffer of one batch
// ([W*H, C, batch] bytes, the reference's packed order == NCHW).  Per batch:
//   1. the producer fills host_slot(i)             (host; after wait_slot_free(i))
//   2. submit(i, ...) enqueues the copy on the copy stream and, behind an event, the conversion on the
//      caller's stream; nothing blocks the host
//   3. the caller's later kernels on its stream see the converted batch in `y`
class ImageBatchStager {
 public:
  ImageBatchStager(size_t inner, size_t channels, size_t batch, int depth = 2)
      : inner_(inner), channels_(channels), batch_(batch), bytes_(inner * channels * batch) {
    if (depth < 1) throw std::invalid_argument("ImageBatchStager: depth must be at least 1");
    (void)sz2uint(bytes_);
    for (int i = 0; i < depth; ++i) slots_.push_back(std::make_unique<Slot>(bytes_));
  }
  ~ImageBatchStager() {
    // copies into the device slots and conversions still reading them finish before the slots are freed
    (void)hipStreamSynchronize(copy_stream_.get());
    for (auto &s : slots_) {
      if (s->in_flight) (void)hipEventSynchronize(s->consumed.get());
    }
  }
  ImageBatchStager(const ImageBatchStager &) = delete;
  ImageBatchStager &operator=(const ImageBatchStager &) = delete;

  int depth() const { return int(slots_.size()); }
  size_t batch_bytes() const { return bytes_; }
  uint8_t *host_slot(int i) { return slots_.at(size_t(i))->host.data(); }

  // Blocks the host until slot i's previous copy has left the pinned buffer (it may then be refilled).
  void wait_slot_free(int i) {
    Slot &s = *slots_.at(size_t(i));
    if (s.in_flight) detail::hip_ok(hipEventSynchronize(s.copied.get()), "wait_slot_free");
  }

  // y[w, c, n] = fma(scale[c], float(q[w, c, n]), shift[c]); scale / shift are device arrays of `channels` floats.
  void submit(int i, const GPUDeviceConn &conn, const float *scale, const float *shift, DeviceArray<float> &y) {
    Slot &s = *slots_.at(size_t(i));
    detail::require_packed("ImageBatchStager::submit", y);
    if (y.shape.flat_len() != bytes_) throw std::invalid_argument("ImageBatchStager::submit: output size");
    hipStream_t compute = reinterpret_cast<hipStream_t>(conn.cuda_stream());
    hipStream_t copy = copy_stream_.get();
    // the device slot may still be read by the conversion submitted from it last time
    if (s.in_flight) detail::hip_ok(hipStreamWaitEvent(copy, s.consumed.get(), 0), "hipStreamWaitEvent");
    detail::hip_ok(hipMemcpyAsync(s.dev.data(), s.host.data(), bytes_, hipMemcpyHostToDevice, copy), "hipMemcpyAsync");
    detail::hip_ok(hipEventRecord(s.copied.get(), copy), "hipEventRecord");
    detail::hip_ok(hipStreamWaitEvent(compute, s.copied.get(), 0), "hipStreamWaitEvent");
    anode_gpu_bcast_dequantize_u8_I1b_I2abc_Oabc_packed_f32(sz2uint(inner_), sz2uint(channels_), sz2uint(batch_), scale,
                                                            shift, s.dev.data(), y.as_mut_dptr(),
                                                            conn.cuda_kernel_config(), conn.cuda_stream());
    detail::hip_ok(hipEventRecord(s.consumed.get(), compute), "hipEventRecord");
    s.in_flight = true;
  }

 private:
  struct Slot {
    explicit Slot(size_t bytes) : host(bytes), dev(bytes) {}
    PinnedBuffer<uint8_t> host;
    DeviceBuffer<uint8_t> dev;
    Event copied, consumed;
    bool in_flight = false;
  };
  size_t inner_, channels_, batch_, bytes_;
  CopyStream copy_stream_;
  std::vector<std::unique_ptr<Slot>> slots_;
};

// ---------------------------------------------------------------------------
// predictions out: device arg-max, one u32 per row to the host
// ---------------------------------------------------------------------------

class LogitsArgMaxReader {
 public:
  explicit LogitsArgMaxReader(size_t max_rows) : host_(max_rows), dev_(max_rows), rows_(max_rows) {}
  LogitsArgMaxReader(const LogitsArgMaxReader &) = delete;
  LogitsArgMaxReader &operator=(const LogitsArgMaxReader &) = delete;

  // logits is [K, rows] (K fastest).  Returns the predicted class of every row; valid until the next call.
  const uint32_t *read(const GPUDeviceConn &conn, const DeviceArray<float> &logits) {
    detail::require_packed("LogitsArgMaxReader::read", logits);
    const size_t rows = logits.shape.batch;
    if (rows > rows_) throw std::invalid_argument("LogitsArgMaxReader::read: more rows than the reader was built for");
    const size_t K = rows ? logits.shape.flat_len() / rows : 0;
    hipStream_t s = reinterpret_cast<hipStream_t>(conn.cuda_stream());
    anode_gpu_arg_max_packed_u32(sz2uint(K), sz2uint(rows), logits.as_dptr(), dev_.data(), conn.cuda_kernel_config(),
                                 conn.cuda_stream());
    detail::hip_ok(hipMemcpyAsync(host_.data(), dev_.data(), rows * sizeof(uint32_t), hipMemcpyDeviceToHost, s), "hipMemcpyAsync");
    detail::hip_ok(hipStreamSynchronize(s), "hipStreamSynchronize");
    return host_.data();
  }

 private:
  PinnedBuffer<uint32_t> host_;
  DeviceBuffer<uint32_t> dev_;
  size_t rows_;
};

}  // namespace anode_host
