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

// The same output walked as the flat array it is: a thread writes one aligned 16-byte group of y (four consecutive
// pixels of one class, or, for the one group per plane that lies across a plane's end where P is not a multiple of
// four, pixels of two planes) and fetches the labels of its pixels, which every class of a sample asks for again,
// from the caches.  The stores are aligned whatever P is, and streamed.
template <int NT>
__global__ __launch_bounds__(kBlock) void one_hot_flat_kernel(uint32_t P, uint32_t K, uint32_t len, FastDiv div_p,
                                                              FastDiv div_k, const uint32_t *__restrict__ cat,
                                                              float *__restrict__ y) {
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;      // 64-bit: index + stride can pass 2^32
  const uint64_t total_groups = (uint64_t(len) + 3u) / 4u;  // (len + 3 can pass 2^32)
  for (uint64_t g64 = uint64_t(blockIdx.x) * kBlock + threadIdx.x; g64 < total_groups; g64 += stride) {
    const uint32_t e = uint32_t(g64) * 4u;  // the group's first element: below len
    uint32_t plane, r;                      // plane = n * K + k, r = the pixel
    div_p.divmod(e, plane, r);
    const uint32_t n0 = div_k.div(plane);
    const uint32_t k0 = plane - n0 * K;
    if (r + 4u <= P && uint64_t(e) + 4u <= len) {
      const u32x4 lab = load_stream<0>(reinterpret_cast<const u32x4 *>(cat + (size_t(n0) * P + r)));
      store_stream<NT>(reinterpret_cast<f32x4 *>(y + e),
                       f32x4{lab.x == k0 ? 1.0f : 0.0f, lab.y == k0 ? 1.0f : 0.0f, lab.z == k0 ? 1.0f : 0.0f,
                             lab.w == k0 ? 1.0f : 0.0f});
    } else {
      // across the end of a plane (P >= 16: of one plane only) or of the array: element by element, the labels
      // requested before any is used
      uint32_t kk[4], label[4];
      bool in[4];
#pragma unroll
      for (uint32_t w = 0; w < 4u; ++w) {
        in[w] = uint64_t(e) + w < len;
        const bool next = r + w >= P;  // the element belongs to the next plane
        const uint32_t rr = next ? r + w - P : r + w;
        uint32_t k = next ? k0 + 1u : k0, n = n0;
        if (k == K) {                  // ... which is the first plane of the next sample
          k = 0u;
          n += 1u;
        }
        kk[w] = k;
        label[w] = in[w] ? cat[size_t(n) * P + rr] : 0u;
      }
#pragma unroll
      for (uint32_t w = 0; w < 4u; ++w) {
        if (in[w]) y[e + w] = label[w] == kk[w] ? 1.0f : 0.0f;
      }
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
  if ((dim0 % 4 == 0 && dim0 >= 16) || dim0 >= 512) {
    // [4224, 21] 5.3 -> 6.2 TB/s, [1024, 100] 6.0 -> 6.8, [524288, 19] 5.1 -> 6.5, [48, 10] 5.0 -> 6.9 against the
    // kernel below, whose threads write their pixels' K planes; planes that are not whole 16-byte groups, against one
    // pixel per thread: [4225, 21] 3.6 -> 5.3, [65535, 4] 3.4 -> 5.0, [513, 19] 3.7 -> 3.9 (shorter ones: most waves
    // then hold a group that lies across the end of a plane, [169, 19] 3.2 against 3.6 below)
    const int nt = policy_for_outputs(stream_policy(size_t(len) * sizeof(float), tuning().nontemporal), y);
    with_stream_policy(nt, [&](auto policy) {
      one_hot_flat_kernel<decltype(policy)::value><<<stream_grid((uint64_t(len) + 3u) / 4u, 1), kBlock, 0, s>>>(
          dim0, cat_dim1, len, FastDiv(dim0), FastDiv(cat_dim1), x, y);
    });
  } else if (dim0 % 4 == 0) {  // (16-byte accesses from any 4-byte aligned address; the stores are ordinary ones)
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
