// Elementwise maps over flat packed arrays: the flat_map family, the two-input
// join, u8 -> 32-bit widening (upcast, dequantize) and the additive f32 -> u8
// quantiser.
//
// Data path: every lane moves 16 bytes per access (global_load/store_dwordx4) and
// consecutive lanes touch consecutive 16-byte groups.  Arrays may start at any
// element: up to 31 head elements are peeled so that the stores start on a
// 128-byte line, and the loads are issued where the inputs lie.  All maps
// read an element before writing the same index, so an output that aliases an
// input at equal index is safe.
#include "common.hpp"

#include <cmath>

namespace anode {
namespace {

// ---- functors: out = f(a[, b]) -------------------------------------------------
// Arithmetic follows routines_gpu/flat_map.cu and flat_join.cu literally; the file
// is compiled with -ffp-contract=off so only the fmaf() written here is fused.

struct CopyMap { __device__ float operator()(float x, float) const { return x; } };
struct ModulusMap { __device__ float operator()(float x, float) const { return fabsf(x); } };
struct SquareMap { __device__ float operator()(float x, float) const { return x * x; } };
struct SqrtMap { __device__ float operator()(float x, float) const { return sqrtf(x); } };
// ReLU by multiplication (flat_map.cu:175-178): negative x gives -0, -inf gives NaN.
struct PositiveClipMap { __device__ float operator()(float x, float) const { return x * float(x > 0.0f); } };
struct LogisticMap { __device__ float operator()(float x, float) const { return 1.0f / (1.0f + expf(-x)); } };
struct UnitStepMap { __device__ float operator()(float x, float) const { return float(x > 0.0f); } };
struct NormalCdfMap {
  __device__ float operator()(float x, float) const { return 0.5f * (1.0f + erff(x * 0.7071067811865475f)); }
};
struct TanhMap { __device__ float operator()(float x, float) const { return tanhf(x); } };
// 1 / cosh(x)^2 = 4t / (1 + t)^2 with t = exp(-2|x|): one exponential, no overflow for any x (coshf costs several
// times more and the kernel stops being bandwidth-bound); within a few ulp of 1 / (coshf(x) * coshf(x))
struct Rcosh2Map {
  __device__ float operator()(float x, float) const {
    const float t = expf(-2.0f * fabsf(x));
    const float d = 1.0f + t;
    return 4.0f * t / (d * d);
  }
};
// Whitelisted for binding by the reference (build.rs:101-102) but left without a wrapper there; functor bodies at
// flat_map.cu:242-278.  x <= 0 and NaN take the else branch.
struct LogPositiveClipMap {
  __device__ float operator()(float x, float) const { return (x > 0.0f) ? logf(x) : -__builtin_huge_valf(); }
};
struct PositiveReciprocalMap {
  __device__ float operator()(float x, float) const { return (x > 0.0f) ? 1.0f / x : 0.0f; }
};
struct LeakyReluMap {
  float c;
  __device__ float operator()(float x, float) const {
    const float mask = float(x > 0.0f);
    return fmaf(1.0f - mask, c, mask) * x;
  }
};
// backward maps: a = dy, b = y
struct LeakyReluBwdMap {
  float c;
  __device__ float operator()(float dy, float y) const {
    const float mask = float(y > 0.0f);
    return fmaf(1.0f - mask, c, mask) * dy;
  }
};
struct PositiveClipBwdMap { __device__ float operator()(float dy, float y) const { return dy * float(y > 0.0f); } };
struct LogisticBwdMap { __device__ float operator()(float dy, float y) const { return dy * y * (1.0f - y); } };
// flat_join.cu:31-35: a = x1, b = x2
struct CopyUnitStepProductJoin { __device__ float operator()(float x1, float x2) const { return x1 * float(x2 > 0.0f); } };

template <typename Op>
__device__ inline f32x4 apply_vec(const Op &op, f32x4 a, f32x4 b) {
  f32x4 r;
  r.x = op(a.x, b.x);
  r.y = op(a.y, b.y);
  r.z = op(a.z, b.z);
  r.w = op(a.w, b.w);
  return r;
}

// `head` single elements, then n_groups groups of four, then `tail` single elements; the single elements are
// handled by workgroup 0.  The host picks head so that the groups of `out_` start on a 128-byte line; the inputs
// are read where they lie (4-byte aligned 16-byte loads).
template <int NIN, int NT, typename Op>
__global__ __launch_bounds__(kBlock) void flat_map_kernel(uint32_t head, uint32_t n_groups, uint32_t tail, Op op,
                                                          const float *a_, const float *b_, float *out_) {
  // no __restrict__: out_ may alias a_ or b_ at equal index
  const f32x4 *a = reinterpret_cast<const f32x4 *>(a_ + head);
  const f32x4 *b = reinterpret_cast<const f32x4 *>(b_ + head);
  f32x4 *out = reinterpret_cast<f32x4 *>(out_ + head);
  // one 16-byte group per thread on a full grid: measured faster on MI355X than any unrolled persistent loop
  // (two or four groups per thread on a correspondingly smaller grid, all their loads in flight together, run at
  // 6.1 TB/s against 6.65 for the copy of 822 MB arrays); the loop only runs more than once under the grid cap of
  // the tuning hook
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;  // 64-bit: index + stride can pass 2^32
  for (uint64_t g = uint64_t(blockIdx.x) * kBlock + threadIdx.x; g < n_groups; g += stride) {
    const f32x4 va = load_stream<NT>(&a[g]);
    const f32x4 vb = (NIN == 2) ? load_stream<NT>(&b[g]) : va;
    store_stream<NT>(&out[g], apply_vec(op, va, vb));
  }
  if (blockIdx.x == 0 && threadIdx.x < head + tail) {
    const uint32_t i = threadIdx.x < head ? threadIdx.x : n_groups * 4u + threadIdx.x;  // (head + 4 * n_groups + (t - head))
    const float x = a_[i];
    const float y = (NIN == 2) ? b_[i] : x;
    out_[i] = op(x, y);
  }
}

template <int NIN, typename Op>
void launch_flat_map(const char *symbol, uint32_t len, Op op, const float *a, const float *b, float *out,
                     CUstream_st *stream) {
  if (len == 0) return;
  const Tuning &t = tuning();
  hipStream_t s = as_stream(stream);
  const int nt = stream_policy(size_t(len) * sizeof(float), t.nontemporal);
  const uint32_t head = head_to_align_line(out, len);
  const uint32_t groups = (len - head) / 4, tail = (len - head) % 4;
  with_stream_policy(nt, [&](auto policy) {
    flat_map_kernel<NIN, decltype(policy)::value, Op>
        <<<stream_grid(groups ? groups : 1, 1), kBlock, 0, s>>>(head, groups, tail, op, a, b, out);
  });
  note_launch(symbol);
}

// ---- u8 -> 32-bit widening -----------------------------------------------------

struct UpcastOp {
  typedef uint32_t out_t;
  typedef u32x4 out4_t;
  __device__ uint32_t operator()(uint32_t q) const { return q; }
};
// quantize.cu:30-32: scale = (hi - lo) / 255; y = float(x) * scale + lo as one fma
struct DequantizeOp {
  typedef float out_t;
  typedef f32x4 out4_t;
  float scale, lo;
  __device__ float operator()(uint32_t q) const { return fmaf(float(q), scale, lo); }
};

// Each lane loads 16 codes in one access, the wave re-deals the dwords through LDS, and each lane converts the
// four dwords it is dealt, so that every load (1 KiB) and every store (four of 1 KiB) of the wave is contiguous.
// One tile per workgroup, 4096 codes.  Measured 34.7 us against 35.8 us for a form with one dword per lane at
// [256,3,224,224].  `head` elements (0 to 31) come first, one per thread of workgroup 0, so that the groups of y
// start on a 128-byte line wherever y lies; the codes are read where they lie (byte-aligned 16-byte loads).
template <int NT, typename Op>
__global__ __launch_bounds__(kBlock) void widen_u8x16_kernel(uint32_t head, uint32_t n_dwords, uint32_t tail, Op op,
                                                             const uint8_t *__restrict__ x_,
                                                             typename Op::out_t *__restrict__ y_) {
  typedef typename Op::out4_t O4;
  __shared__ __align__(16) uint32_t lds[kBlock * 4];
  const uint8_t *x = x_ + head;
  const u32x4 *x16 = reinterpret_cast<const u32x4 *>(x);
  O4 *y4 = reinterpret_cast<O4 *>(y_ + head);
  const uint32_t wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const uint64_t g16 = uint64_t(blockIdx.x) * kBlock + threadIdx.x;  // this lane's group of 16 codes
  const uint64_t wave_first = (uint64_t(blockIdx.x) * kBlock + uint64_t(wave) * kWave) * 4u;  // the wave's first dword
  u32x4 v = {0u, 0u, 0u, 0u};
  if (g16 * 4u + 3u < n_dwords) {
    v = load_stream<kNtLoad, 1>(&x16[g16]);  // the codes are read once, whatever the size
  } else if (g16 * 4u < n_dwords) {  // the last, partial group of the array: dword by dword
    const uint32_t *x4 = reinterpret_cast<const uint32_t *>(x);
    for (uint32_t k = 0; k < 4u && g16 * 4u + k < n_dwords; ++k) v[k] = load_stream<0, 1>(&x4[g16 * 4u + k]);
  }
  uint32_t w[4];
  wave_deal_dwords(v, lds + wave * (kWave * 4), w);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint64_t d = wave_first + uint32_t(j) * kWave + lane;
    if (d < n_dwords) {
      O4 r;
      r.x = op(w[j] & 0xffu);
      r.y = op((w[j] >> 8) & 0xffu);
      r.z = op((w[j] >> 16) & 0xffu);
      r.w = op(w[j] >> 24);
      store_stream<NT>(&y4[d], r);
    }
  }
  if (blockIdx.x == 0 && threadIdx.x < head + tail) {
    const uint32_t i = threadIdx.x < head ? threadIdx.x : n_dwords * 4u + threadIdx.x;
    y_[i] = op(uint32_t(x_[i]));
  }
}

template <typename Op>
void launch_widen_u8(const char *symbol, uint32_t len, Op op, const uint8_t *x, typename Op::out_t *y,
                     CUstream_st *stream) {
  if (len == 0) return;
  const Tuning &t = tuning();
  hipStream_t s = as_stream(stream);
  const uint32_t head = head_to_align_line(y, len);
  const uint32_t dwords = (len - head) / 4, tail = (len - head) % 4;
  const uint32_t blocks = (dwords + kBlock * 4 - 1) / (kBlock * 4);
  // the policy looks at the output, which is four times the input
  const int nt = stream_policy(size_t(len) * 4, t.nontemporal);
  with_stream_policy(nt, [&](auto policy) {
    widen_u8x16_kernel<decltype(policy)::value, Op><<<blocks ? blocks : 1, kBlock, 0, s>>>(head, dwords, tail, op, x, y);
  });
  note_launch(symbol);
}

}  // namespace
}  // namespace anode

using namespace anode;

#define ANODE_FLAT_MAP1(SYMBOL, OP)                                                              \
  ANODE_EXPORT void SYMBOL(uint32_t len, const float *x, float *y, const KernelConfig *,       \
                           CUstream_st *stream) {                                                \
    launch_flat_map<1>(#SYMBOL, len, OP{}, x, x, y, stream);                                     \
  }

#define ANODE_FLAT_MAP2(SYMBOL, OP)                                                              \
  ANODE_EXPORT void SYMBOL(uint32_t len, const float *a, const float *b, float *out,            \
                           const KernelConfig *, CUstream_st *stream) {                          \
    launch_flat_map<2>(#SYMBOL, len, OP{}, a, b, out, stream);                                   \
  }

ANODE_FLAT_MAP1(anode_gpu_copy_flat_map_f32, CopyMap)
ANODE_FLAT_MAP1(anode_gpu_modulus_flat_map_f32, ModulusMap)
ANODE_FLAT_MAP1(anode_gpu_square_flat_map_f32, SquareMap)
ANODE_FLAT_MAP1(anode_gpu_sqrt_flat_map_f32, SqrtMap)
ANODE_FLAT_MAP1(anode_gpu_positive_clip_flat_map_f32, PositiveClipMap)
ANODE_FLAT_MAP1(anode_gpu_logistic_flat_map_f32, LogisticMap)
ANODE_FLAT_MAP1(anode_gpu_unit_step_flat_map_f32, UnitStepMap)
ANODE_FLAT_MAP1(anode_gpu_normal_cdf_flat_map_f32, NormalCdfMap)
ANODE_FLAT_MAP1(anode_gpu_tanh_flat_map_f32, TanhMap)
ANODE_FLAT_MAP1(anode_gpu_rcosh2_flat_map_f32, Rcosh2Map)
// additive: named in the reference's bindgen whitelist (build.rs:101-102), never defined there
ANODE_FLAT_MAP1(anode_gpu_log_positive_clip_flat_map_f32, LogPositiveClipMap)
ANODE_FLAT_MAP1(anode_gpu_positive_reciprocal_flat_map_f32, PositiveReciprocalMap)

ANODE_FLAT_MAP2(anode_gpu_positive_clip_flat_map_bwd_f32, PositiveClipBwdMap)
ANODE_FLAT_MAP2(anode_gpu_logistic_flat_map_bwd_f32, LogisticBwdMap)
ANODE_FLAT_MAP2(anode_gpu_M1_copy_map_M2_unit_step_map_R_product_reduce_flat_join_f32, CopyUnitStepProductJoin)

ANODE_EXPORT void anode_gpu_leaky_relu_flat_map_f32(uint32_t len, float c, const float *x, float *y,
                                                    const KernelConfig *, CUstream_st *stream) {
  launch_flat_map<1>("anode_gpu_leaky_relu_flat_map_f32", len, LeakyReluMap{c}, x, x, y, stream);
}

ANODE_EXPORT void anode_gpu_leaky_relu_flat_map_bwd_f32(uint32_t len, float c, const float *dy,
                                                        const float *y, float *dx, const KernelConfig *,
                                                        CUstream_st *stream) {
  launch_flat_map<2>("anode_gpu_leaky_relu_flat_map_bwd_f32", len, LeakyReluBwdMap{c}, dy, y, dx, stream);
}

ANODE_EXPORT void anode_gpu_upcast_u8_packed_u32(uint32_t len, const uint8_t *x, uint32_t *y,
                                                 const KernelConfig *, CUstream_st *stream) {
  launch_widen_u8("anode_gpu_upcast_u8_packed_u32", len, UpcastOp{}, x, y, stream);
}

ANODE_EXPORT void anode_gpu_dequantize_u8_packed_f32(uint32_t len, float lo, float hi, const uint8_t *x,
                                                     float *y, const KernelConfig *, CUstream_st *stream) {
  // the scale is formed on the host exactly as the kernel preamble of
  // quantize.cu:30 forms it: an fp32 subtraction and an fp32 division
  const float scale = (hi - lo) / 255.0f;
  launch_widen_u8("anode_gpu_dequantize_u8_packed_f32", len, DequantizeOp{scale, lo}, x, y, stream);
}
