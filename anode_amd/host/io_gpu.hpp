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

#include "anode_amd/host/ops_gpu.hpp"

#include <hip/hip_runtime.h>

#include <cstring>
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
    detail::hip_ok(hipStreamCreateWithFlags(&copy_stream_, hipStreamNonBlocking), "hipStreamCreate");
    slots_.resize(size_t(depth));
    for (Slot &s : slots_) {
      s.host = new PinnedBuffer<uint8_t>(bytes_);
      detail::hip_ok(hipMalloc(reinterpret_cast<void **>(&s.dev), bytes_ ? bytes_ : 1), "hipMalloc");
      detail::hip_ok(hipEventCreateWithFlags(&s.copied, hipEventDisableTiming), "hipEventCreate");
      detail::hip_ok(hipEventCreateWithFlags(&s.consumed, hipEventDisableTiming), "hipEventCreate");
    }
  }
  ~ImageBatchStager() {
    (void)hipStreamSynchronize(copy_stream_);
    for (Slot &s : slots_) {
      if (s.in_flight) (void)hipEventSynchronize(s.consumed);
      (void)hipEventDestroy(s.copied);
      (void)hipEventDestroy(s.consumed);
      (void)hipFree(s.dev);
      delete s.host;
    }
    (void)hipStreamDestroy(copy_stream_);
  }
  ImageBatchStager(const ImageBatchStager &) = delete;
  ImageBatchStager &operator=(const ImageBatchStager &) = delete;

  int depth() const { return int(slots_.size()); }
  size_t batch_bytes() const { return bytes_; }
  uint8_t *host_slot(int i) { return slots_.at(size_t(i)).host->data(); }

  // Blocks the host until slot i's previous copy has left the pinned buffer (it may then be refilled).
  void wait_slot_free(int i) {
    Slot &s = slots_.at(size_t(i));
    if (s.in_flight) detail::hip_ok(hipEventSynchronize(s.copied), "wait_slot_free");
  }

  // y[w, c, n] = fma(scale[c], float(q[w, c, n]), shift[c]); scale / shift are device arrays of `channels` floats.
  void submit(int i, const GPUDeviceConn &conn, const float *scale, const float *shift, DeviceArray<float> &y) {
    Slot &s = slots_.at(size_t(i));
    detail::require_packed("ImageBatchStager::submit", y);
    if (y.shape.flat_len() != bytes_) throw std::invalid_argument("ImageBatchStager::submit: output size");
    hipStream_t compute = reinterpret_cast<hipStream_t>(conn.cuda_stream());
    // the device slot may still be read by the conversion submitted from it last time
    if (s.in_flight) detail::hip_ok(hipStreamWaitEvent(copy_stream_, s.consumed, 0), "hipStreamWaitEvent");
    detail::hip_ok(hipMemcpyAsync(s.dev, s.host->data(), bytes_, hipMemcpyHostToDevice, copy_stream_), "hipMemcpyAsync");
    detail::hip_ok(hipEventRecord(s.copied, copy_stream_), "hipEventRecord");
    detail::hip_ok(hipStreamWaitEvent(compute, s.copied, 0), "hipStreamWaitEvent");
    anode_gpu_bcast_dequantize_u8_I1b_I2abc_Oabc_packed_f32(sz2uint(inner_), sz2uint(channels_), sz2uint(batch_), scale,
                                                            shift, s.dev, y.as_mut_dptr(), conn.cuda_kernel_config(),
                                                            conn.cuda_stream());
    detail::hip_ok(hipEventRecord(s.consumed, compute), "hipEventRecord");
    s.in_flight = true;
  }

 private:
  struct Slot {
    PinnedBuffer<uint8_t> *host = nullptr;
    uint8_t *dev = nullptr;
    hipEvent_t copied = nullptr, consumed = nullptr;
    bool in_flight = false;
  };
  size_t inner_, channels_, batch_, bytes_;
  hipStream_t copy_stream_ = nullptr;
  std::vector<Slot> slots_;
};

// ---------------------------------------------------------------------------
// predictions out: device arg-max, one u32 per row to the host
// ---------------------------------------------------------------------------

class LogitsArgMaxReader {
 public:
  explicit LogitsArgMaxReader(size_t max_rows) : host_(max_rows), rows_(max_rows) {
    detail::hip_ok(hipMalloc(reinterpret_cast<void **>(&dev_), (max_rows ? max_rows : 1) * sizeof(uint32_t)), "hipMalloc");
  }
  ~LogitsArgMaxReader() { (void)hipFree(dev_); }
  LogitsArgMaxReader(const LogitsArgMaxReader &) = delete;
  LogitsArgMaxReader &operator=(const LogitsArgMaxReader &) = delete;

  // logits is [K, rows] (K fastest).  Returns the predicted class of every row; valid until the next call.
  const uint32_t *read(const GPUDeviceConn &conn, const DeviceArray<float> &logits) {
    detail::require_packed("LogitsArgMaxReader::read", logits);
    const size_t rows = logits.shape.batch;
    if (rows > rows_) throw std::invalid_argument("LogitsArgMaxReader::read: more rows than the reader was built for");
    const size_t K = rows ? logits.shape.flat_len() / rows : 0;
    hipStream_t s = reinterpret_cast<hipStream_t>(conn.cuda_stream());
    anode_gpu_arg_max_packed_u32(sz2uint(K), sz2uint(rows), logits.as_dptr(), dev_, conn.cuda_kernel_config(),
                                 conn.cuda_stream());
    detail::hip_ok(hipMemcpyAsync(host_.data(), dev_, rows * sizeof(uint32_t), hipMemcpyDeviceToHost, s), "hipMemcpyAsync");
    detail::hip_ok(hipStreamSynchronize(s), "hipStreamSynchronize");
    return host_.data();
  }

 private:
  PinnedBuffer<uint32_t> host_;
  uint32_t *dev_ = nullptr;
  size_t rows_;
};

}  // namespace anode_host
