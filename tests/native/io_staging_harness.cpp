// Native harness for the staging layer (anode_amd/host/io_gpu.hpp): checks the
// pinned, double-buffered image pipeline and the device arg-max reader against
// the CPU oracle, then times them beside the reference's way of doing the same
// job (synchronous pageable copies + a separate operator, src/io_gpu.rs:286-330)
// and prints the host-buffer-inclusive rates as one JSON line.  Test infrastructure.
#include "anode_amd/host/io_gpu.hpp"
#include "tests/native/ops_gpu.hpp"

#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

using namespace anode_host;

extern "C" {
// oracle/anode_oracle.c
void oracle_bcast_dequantize_u8(uint32_t, uint32_t, uint32_t, const float *, const float *, const uint8_t *, float *);
void oracle_dequantize_u8_f32ref(uint32_t, float, float, const uint8_t *, float *);
void oracle_arg_max_rows(uint32_t, uint32_t, const float *, uint32_t *);
}

static int g_checks = 0, g_failed = 0;

#define HIP_OK(x)                                                                       \
  do {                                                                                  \
    hipError_t e_ = (x);                                                                \
    if (e_ != hipSuccess) {                                                             \
      std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);        \
      std::exit(2);                                                                     \
    }                                                                                   \
  } while (0)

static void check(bool ok, const char *what) {
  ++g_checks;
  if (!ok) ++g_failed;
  std::printf("%s %s\n", ok ? "ok  " : "FAIL", what);
  std::fflush(stdout);
}

static uint32_t lcg(uint32_t &s) {
  s = s * 1664525u + 1013904223u;
  return s >> 8;
}

static double now_s() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

template <typename T>
struct DevMem {
  T *p = nullptr;
  explicit DevMem(size_t n) { HIP_OK(hipMalloc(reinterpret_cast<void **>(&p), (n ? n : 1) * sizeof(T))); }
  ~DevMem() { (void)hipFree(p); }
};

int main() {
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  GPUDeviceConn conn;
  conn.stream = stream;

  const std::vector<float> h_scale = {1.0f / (255.0f * 0.229f), 1.0f / (255.0f * 0.224f), 1.0f / (255.0f * 0.225f)};
  const std::vector<float> h_shift = {-0.485f / 0.229f, -0.456f / 0.224f, -0.406f / 0.225f};
  DevMem<float> scale(3), shift(3);
  HIP_OK(hipMemcpy(scale.p, h_scale.data(), 12, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(shift.p, h_shift.data(), 12, hipMemcpyHostToDevice));

  // ---- correctness: five batches through a two-slot stager, each into its own output ----
  {
    const size_t inner = 56 * 56 + 1, C = 3, N = 16, n = inner * C * N;  // odd inner: groups straddle channels
    ImageBatchStager stager(inner, C, N, 2);
    const int batches = 5;
    std::vector<std::vector<uint8_t>> src(batches, std::vector<uint8_t>(n));
    std::vector<DevMem<float> *> out;
    uint32_t seed = 1;
    bool ok = true;
    for (int b = 0; b < batches; ++b) {
      for (auto &v : src[size_t(b)]) v = uint8_t(lcg(seed));
      out.push_back(new DevMem<float>(n));
      const int slot = b % stager.depth();
      stager.wait_slot_free(slot);
      std::memcpy(stager.host_slot(slot), src[size_t(b)].data(), n);
      auto y = obatch3d(out.back()->p, inner, 1, C, N);
      stager.submit(slot, conn, scale.p, shift.p, y);
    }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<float> got(n), want(n);
    for (int b = 0; b < batches; ++b) {
      HIP_OK(hipMemcpy(got.data(), out[size_t(b)]->p, n * sizeof(float), hipMemcpyDeviceToHost));
      oracle_bcast_dequantize_u8(uint32_t(inner), uint32_t(C), uint32_t(N), h_scale.data(), h_shift.data(),
                                 src[size_t(b)].data(), want.data());
      ok = ok && std::memcmp(got.data(), want.data(), n * sizeof(float)) == 0;
      delete out[size_t(b)];
    }
    check(ok, "ImageBatchStager: five batches through two slots, bit-exact against the oracle");
  }

  // ---- correctness: sync_copy_mem / sync_dump_mem round trip and the arg-max reader ----
  const size_t K = 1000, R = 256;
  std::vector<float> logits(K * R);
  {
    uint32_t seed = 7;
    for (auto &v : logits) v = float(lcg(seed) % 2001u) * 0.01f - 10.0f;  // coarse grid: ties are common
    logits[5 * K + 3] = NAN;
    for (size_t k = 0; k < K; ++k) logits[9 * K + k] = -INFINITY;
    DevMem<float> d(K * R);
    auto a = obatch1d(d.p, K, R);
    sync_copy_mem(a, logits.data(), conn);
    std::vector<float> back(K * R);
    sync_dump_mem(a, back.data(), conn);
    check(std::memcmp(back.data(), logits.data(), K * R * sizeof(float)) == 0, "sync_copy_mem / sync_dump_mem round trip");
    LogitsArgMaxReader reader(R);
    const uint32_t *pred = reader.read(conn, a);
    std::vector<uint32_t> want(R);
    oracle_arg_max_rows(uint32_t(K), uint32_t(R), logits.data(), want.data());
    bool ok = true;
    for (size_t r = 0; r < R; ++r) ok = ok && pred[r] == want[r];
    check(ok, "LogitsArgMaxReader equals the host rule (ties, NaN, all -inf)");
  }

  // ---- timing: u8 [224*224, 3, 256] in, f32 out ----
  const size_t inner = 224 * 224, C = 3, N = 256, n = inner * C * N;
  const int reps = 20;
  double t_ref = 0.0, t_pipe = 0.0, t_pipe_fill = 0.0;
  {
    std::vector<uint8_t> pageable(n);
    uint32_t seed = 3;
    for (size_t i = 0; i < n; i += 97) pageable[i] = uint8_t(lcg(seed));
    DevMem<uint8_t> dq(n);
    DevMem<float> dy(n);
    auto qa = obatch3d(dq.p, 224, 224, C, N);
    auto ya = obatch3d(dy.p, 224, 224, C, N);
    // the reference's sequence: synchronous copy from pageable memory, then the dequantize operator
    for (int r = 0; r < reps + 2; ++r) {
      if (r == 2) t_ref = now_s();
      sync_copy_mem(qa, pageable.data(), conn);
      DequantizeOp::apply(WriteCap::Assign, conn, 0.0f, 1.0f, qa, ya);
      HIP_OK(hipStreamSynchronize(stream));
    }
    t_ref = (now_s() - t_ref) / reps;

    ImageBatchStager stager(inner, C, N, 2);
    for (int s = 0; s < stager.depth(); ++s) std::memcpy(stager.host_slot(s), pageable.data(), n);
    // slots already hold the data (a decoder writes into them directly)
    for (int r = 0; r < reps + 2; ++r) {
      if (r == 2) {
        HIP_OK(hipStreamSynchronize(stream));
        t_pipe = now_s();
      }
      const int slot = r % stager.depth();
      stager.wait_slot_free(slot);
      stager.submit(slot, conn, scale.p, shift.p, ya);
    }
    HIP_OK(hipStreamSynchronize(stream));
    t_pipe = (now_s() - t_pipe) / reps;
    // including a host memcpy from pageable memory into the slot (a loader that cannot write in place)
    for (int r = 0; r < reps + 2; ++r) {
      if (r == 2) {
        HIP_OK(hipStreamSynchronize(stream));
        t_pipe_fill = now_s();
      }
      const int slot = r % stager.depth();
      stager.wait_slot_free(slot);
      std::memcpy(stager.host_slot(slot), pageable.data(), n);
      stager.submit(slot, conn, scale.p, shift.p, ya);
    }
    HIP_OK(hipStreamSynchronize(stream));
    t_pipe_fill = (now_s() - t_pipe_fill) / reps;
  }

  // ---- timing: predictions of [1000, 256] logits ----
  double t_arg_ref = 0.0, t_arg_dev = 0.0;
  {
    DevMem<float> d(K * R);
    auto a = obatch1d(d.p, K, R);
    sync_copy_mem(a, logits.data(), conn);
    std::vector<float> back(K * R);
    std::vector<uint32_t> pred(R);
    const int areps = 200;
    for (int r = 0; r < areps + 5; ++r) {
      if (r == 5) t_arg_ref = now_s();
      sync_dump_mem(a, back.data(), conn);
      for (size_t i = 0; i < R; ++i) pred[i] = uint32_t(anode_host_arg_max_f32(back.data() + i * K, K));
    }
    t_arg_ref = (now_s() - t_arg_ref) / areps;
    LogitsArgMaxReader reader(R);
    for (int r = 0; r < areps + 5; ++r) {
      if (r == 5) t_arg_dev = now_s();
      (void)reader.read(conn, a);
    }
    t_arg_dev = (now_s() - t_arg_dev) / areps;
  }

  check(anode_gpu_take_last_error() == 0, "no launch error recorded");
  std::printf(
      "{\"staging\": {\"image_batch\": \"u8 [256,3,224,224] -> f32\", \"bytes_in\": %zu, \"bytes_out\": %zu, "
      "\"reference_way_ms\": %.3f, \"reference_way_in_gbps\": %.2f, \"pinned_pipeline_ms\": %.3f, "
      "\"pinned_pipeline_in_gbps\": %.2f, \"pinned_pipeline_with_host_fill_ms\": %.3f, "
      "\"logits\": \"f32 [256,1000]\", \"argmax_reference_way_us\": %.1f, \"argmax_device_us\": %.1f}}\n",
      n, n * sizeof(float), t_ref * 1e3, double(n) / t_ref / 1e9, t_pipe * 1e3, double(n) / t_pipe / 1e9, t_pipe_fill * 1e3,
      t_arg_ref * 1e6, t_arg_dev * 1e6);
  HIP_OK(hipStreamDestroy(stream));
  std::printf("%s: %d checks, %d failed\n", g_failed ? "FAILED" : "ALL PASS", g_checks, g_failed);
  return g_failed ? 1 : 0;
}
