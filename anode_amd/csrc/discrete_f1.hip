// One-hot expansion of categorical labels and the smooth negative F1 loss.
#include "chan_map.hpp"
#include "chan_reduce.hpp"
#include "common.hpp"

#include <type_traits>

namespace anode {
namespace {

// discrete.cu:21-46  y[p,k,n] = (label[p + P*n] == k) ? 1 : 0 over a packed
// [P, K, N] output.  A thread reads the labels of W consecutive pixels once and
// writes their K outputs, 16 bytes per store, coalesced across the wave.
template <int W, int NT>
__global__ __launch_bounds__(kBlock) void one_hot_kernel(uint32_t P, uint32_t K, uint32_t total_groups,
                                                         FastDiv div_gps, const uint32_t *__restrict__ cat,
                                                         float *__restrict__ y) {
  typedef typename std::conditional<W == 4, u32x4, uint32_t>::type U;
  typedef typename std::conditional<W == 4, f32x4, float>::type V;
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;  // 64-bit: index + stride can pass 2^32
  for (uint64_t g = uint64_t(blockIdx.x) * kBlock + threadIdx.x; g < total_groups; g += stride) {
    uint32_t n, r;
    div_gps.divmod(uint32_t(g), n, r);  // g < total_groups, which fits 32 bits
    const uint32_t p = r * uint32_t(W);
    const U lab = load_stream<0>(reinterpret_cast<const U *>(cat + (size_t(p) + size_t(P) * n)));
    const size_t base = size_t(p) + size_t(P) * K * n;
#pragma unroll 4
    for (uint32_t k = 0; k < K; ++k) {
      V v;
      if constexpr (W == 4) {
        v = f32x4{lab.x == k ? 1.0f : 0.0f, lab.y == k ? 1.0f : 0.0f, lab.z == k ? 1.0f : 0.0f,
                  lab.w == k ? 1.0f : 0.0f};
      } else {
        v = (lab == k) ? 1.0f : 0.0f;
      }
      store_stream<NT>(reinterpret_cast<V *>(y + base + size_t(P) * k), v);
    }
  }
}

// f1.cu:23-71 as a per-channel reduction over [S = dim0, C = K*N, 1]:
//   y[k,n] = -(2 * sum x*t + eps) / (sum (x + t) + eps)
struct F1Reduce {
  static constexpr int NIN = 2, NACC = 2;  // a = x, b = target
  struct Param {};
  float *y;
  double eps;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ void term(const Param &, float a, float b, double &s0, double &s1, double &) const {
    s0 = fma(double(a), double(b), s0);
    s1 += double(a) + double(b);
  }
  __device__ void finalize(uint32_t c, double s0, double s1, double) const { y[c] = float(-(2.0 * s0 + eps) / (s1 + eps)); }
};

// f1.cu:89-115 as a channel-indexed map over [S = dim0, C = K*N, 1]:
//   dx = dy[k,n] * -(2 t (t + eps) - eps) / (x + t + eps)^2      (a = x, b = target)
struct F1BwdMap {
  const float *dy;
  float eps;
  struct Param { float dy; };
  __device__ Param load(uint32_t c) const { return Param{dy[c]}; }
  __device__ float value(const Param &p, float x, float tg, uint32_t) const {
    const float numer = fmaf(2.0f * tg, tg + eps, -eps);
    const float denom = x + tg + eps;
    return p.dy * -numer / (denom * denom);
  }
  __device__ float accum(const Param &p, float x, float tg, uint32_t s, float old) const {
    return old + value(p, x, tg, s);
  }
};

}  // namespace
}  // namespace anode

using namespace anode;

ANODE_EXPORT void anode_gpu_discrete_one_hot_3d1_packed_f32(uint32_t dim0, uint32_t cat_dim1, uint32_t dim2,
                                                            const uint32_t *x, float *y, const KernelConfig *,
                                                            CUstream_st *stream) {
  const uint32_t len = checked_len(dim0, cat_dim1, dim2, __func__);
  if (len == 0) return;
  hipStream_t s = as_stream(stream);
  if (dim0 % 4 == 0) {  // (16-byte accesses from any 4-byte aligned address; the stores are ordinary ones)
    const uint32_t gps = dim0 / 4, total = gps * dim2;
    // ordinary stores: with streaming stores this kernel, which writes K planes per thread, measured 15 % slower
    one_hot_kernel<4, 0><<<stream_grid(total, 1), kBlock, 0, s>>>(dim0, cat_dim1, total, FastDiv(gps), x, y);
  } else {
    const uint32_t total = dim0 * dim2;
    one_hot_kernel<1, 0><<<stream_grid(total, 1), kBlock, 0, s>>>(dim0, cat_dim1, total, FastDiv(dim0), x, y);
  }
  note_launch(__func__);
}

ANODE_EXPORT void anode_gpu_smooth_negative_f1_loss_3d1_packed_f32(uint32_t dim0, uint32_t cat_dim1, uint32_t dim2,
                                                                   float epsilon, const float *x,
                                                                   const float *target, float *y,
                                                                   const KernelConfig *cfg, CUstream_st *stream) {
  require_pow2_block(cfg, __func__);
  const uint32_t rows = checked_len(cat_dim1, dim2, 1, __func__);
  launch_chan_reduce(__func__, dim0, rows, 1, F1Reduce{y, double(epsilon)}, x, target, stream);
}

ANODE_EXPORT void anode_gpu_smooth_negative_f1_loss_3d1_bwd_packed_f32(uint32_t dim0, uint32_t cat_dim1,
                                                                       uint32_t dim2, float epsilon,
                                                                       const float *dy, const float *x,
                                                                       const float *target, float *dx,
                                                                       const KernelConfig *, CUstream_st *stream) {
  const uint32_t rows = checked_len(cat_dim1, dim2, 1, __func__);
  launch_chan_map<2, false>(__func__, dim0, rows, 1, F1BwdMap{dy, epsilon}, x, target, dx, stream);
}
