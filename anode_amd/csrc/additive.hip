// Entry points that have no kernel in the reference but sit directly on either
// side of the hot path: the inverse of dequantize, the per-channel affine and
// channel sums that the reference only declares (commented out in
// routines_gpu/lib.h:195-249, 406-430), single-pass batch statistics, fused
// batch-norm forward/backward, running averages and arg-max.  They reuse the
// map / reduce templates of the reference ABI kernels.
#include "chan_map.hpp"
#include "chan_reduce.hpp"
#include "common.hpp"

#include <cmath>
#include <cstdio>
#include <mutex>

namespace anode {
namespace {

struct Empty {};

// ---------------------------------------------------------------------------
// f32 -> u8 quantisation: q = clamp(rint((x - lo) / scale), 0, 255), NaN -> 0,
// scale = (hi - lo) / 255; rint rounds half to even.  Inverse of dequantize.
// ---------------------------------------------------------------------------
__device__ inline uint32_t quantize_one(float x, float lo, float scale) {
  float q = rintf((x - lo) / scale);
  q = (q >= 0.0f) ? q : 0.0f;  // also catches NaN
  q = (q > 255.0f) ? 255.0f : q;
  return uint32_t(q);
}

// 16 bytes per lane on both sides: lane l of a wave loads the 16-byte groups j*64 + l (j = 0..3) of the wave's 256,
// packs each to a dword, and the wave gathers the dwords through LDS so that each lane stores 16 consecutive bytes:
// four 1 KiB loads and one 1 KiB store per wave, all contiguous, all four loads of a thread in flight together (the
// input is read once, hence non-temporal).  One tile per workgroup, 4096 elements.  Measured 34.5 us at
// [256,3,224,224] (57 us with one 16-byte load and one 4-byte store per thread).  `head` elements (0 to 127) come
// first, one per thread of workgroup 0, so that the stores start on a 128-byte line wherever y lies; x is
// read where it lies.
__global__ __launch_bounds__(kBlock) void quantize_u8x16_kernel(uint32_t head, uint32_t n_groups, uint32_t tail,
                                                                float lo, float scale, const float *__restrict__ x_,
                                                                uint8_t *__restrict__ y_) {
  __shared__ __align__(16) uint32_t lds[kBlock * 4];
  const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x_ + head);
  uint32_t *y4 = reinterpret_cast<uint32_t *>(y_ + head);
  const uint32_t wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const uint64_t wave_first = (uint64_t(blockIdx.x) * kBlock + uint64_t(wave) * kWave) * 4u;  // first group = first output dword
  f32x4 v[4] = {};
  if (n_groups != 0u) {  // (fewer than four elements: only the single elements below have work)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // unconditional (a group past the end reads the last group again; its code is never stored): with a branch
      // round each load the compiler waits for the previous load before it issues the next one
      const uint64_t g = wave_first + uint32_t(j) * kWave + lane;
      v[j] = load_stream<kNtLoad>(&x4[g < n_groups ? g : uint64_t(n_groups - 1u)]);
    }
  }
  uint32_t d[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    d[j] = quantize_one(v[j].x, lo, scale) | (quantize_one(v[j].y, lo, scale) << 8) |
           (quantize_one(v[j].z, lo, scale) << 16) | (quantize_one(v[j].w, lo, scale) << 24);
  }
  const u32x4 out = wave_gather_dwords(d, lds + wave * (kWave * 4));
  const uint64_t first = wave_first + uint64_t(lane) * 4u;  // this lane's first output dword
  if (first + 3u < n_groups) {
    *reinterpret_cast<u32x4 *>(y4 + first) = out;
  } else {
    for (uint32_t k = 0; k < 4u && first + k < n_groups; ++k) y4[first + k] = out[k];
  }
  if (blockIdx.x == 0 && threadIdx.x < head + tail) {
    const uint32_t i = threadIdx.x < head ? threadIdx.x : n_groups * 4u + threadIdx.x;
    y_[i] = uint8_t(quantize_one(x_[i], lo, scale));
  }
}

// ---------------------------------------------------------------------------
// per-channel affine maps
// ---------------------------------------------------------------------------

// y = lx[b] * rx  /  y = fma(lx[b], rx, shift[b])
struct BcastMultMap {
  const float *lx;
  struct Param { float l; };
  __device__ Param load(uint32_t c) const { return Param{lx[c]}; }
  __device__ float value(const Param &p, float r, float, uint32_t) const { return p.l * r; }
  __device__ float accum(const Param &p, float r, float, uint32_t, float old) const { return fmaf(p.l, r, old); }
};
struct BcastMultAddMap {
  const float *lx, *shift;
  struct Param { float l, s; };
  __device__ Param load(uint32_t c) const { return Param{lx[c], shift[c]}; }
  __device__ float value(const Param &p, float r, float, uint32_t) const { return fmaf(p.l, r, p.s); }
  __device__ float accum(const Param &p, float r, float, uint32_t, float old) const { return old + fmaf(p.l, r, p.s); }
};
// y = fma(lx, rx, shift), all three per element
struct FlatMultAddMap {
  typedef Empty Param;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ float value3(const Param &, float l, float r, float s, uint32_t) const { return fmaf(l, r, s); }
  __device__ float accum3(const Param &, float l, float r, float s, uint32_t, float old) const {
    return old + fmaf(l, r, s);
  }
};
struct FlatMultMap {
  typedef Empty Param;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ float value(const Param &, float l, float r, uint32_t) const { return l * r; }
  __device__ float accum(const Param &, float l, float r, uint32_t, float old) const { return fmaf(l, r, old); }
};

// u8 codes -> per-channel affine f32: y = fma(scale[b], float(q), shift[b]).  One 16-byte load of 16 codes per
// lane, the wave's dwords re-dealt through LDS (see wave_deal_dwords), each lane converts the four dwords it is
// dealt; the channel of a group's first code is found by exact division, then advanced incrementally.  One tile per
// workgroup, 4096 codes.  `head` elements (0 to 31) come first, one per thread of workgroup 0, so that the groups
// of y start on a 128-byte line wherever y lies; the codes are read where they lie.
// LONG: channels of at least 4096 codes (a workgroup's tile): the tile crosses at most one channel boundary, so its
// two channels and their parameters are found once per workgroup on the scalar unit and every code only compares
// its index with the boundary, instead of a division and two dependent parameter fetches per 16-byte group of y
// (u8 [256,3,224,224] -> f32: 41.8 -> 35 us).
template <int NT, bool LONG>
__global__ __launch_bounds__(kBlock) void bcast_dequantize_u8x16_kernel(uint32_t head, uint32_t n_dwords, uint32_t tail,
                                                                        FastDiv div_s, FastDiv div_c,
                                                                        const float *__restrict__ scale,
                                                                        const float *__restrict__ shift,
                                                                        const uint8_t *__restrict__ x_,
                                                                        float *__restrict__ y_) {
  __shared__ __align__(16) uint32_t lds[kBlock * 4];
  const uint8_t *x = x_ + head;
  const u32x4 *x16 = reinterpret_cast<const u32x4 *>(x);
  f32x4 *y4 = reinterpret_cast<f32x4 *>(y_ + head);
  const uint32_t S = div_s.d, C = div_c.d;
  const uint32_t wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const uint64_t g16 = uint64_t(blockIdx.x) * kBlock + threadIdx.x;
  const uint64_t wave_first = (uint64_t(blockIdx.x) * kBlock + uint64_t(wave) * kWave) * 4u;
  u32x4 v = {0u, 0u, 0u, 0u};
  if (g16 * 4u + 3u < n_dwords) {
    v = load_stream<kNtLoad, 1>(&x16[g16]);
  } else if (g16 * 4u < n_dwords) {
    const uint32_t *x4 = reinterpret_cast<const uint32_t *>(x);
    for (uint32_t k = 0; k < 4u && g16 * 4u + k < n_dwords; ++k) v[k] = load_stream<0, 1>(&x4[g16 * 4u + k]);
  }
  uint32_t w[4];
  wave_deal_dwords(v, lds + wave * (kWave * 4), w);
  if (LONG) {
    // the tile's first code is element e0 of the array; its channel run ends at element `edge`
    const uint32_t e0 = head + blockIdx.x * uint32_t(kBlock * 16);
    uint32_t q0, s0;
    div_s.divmod(e0, q0, s0);
    const uint32_t c0 = q0 - div_c.div(q0) * C, c1 = (c0 + 1 == C) ? 0 : c0 + 1;
    const uint32_t edge = S - s0;  // counted from the tile's first code
    const float a0 = scale[c0], b0 = shift[c0], a1 = scale[c1], b1 = shift[c1];  // uniform: scalar loads
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint64_t d = wave_first + uint32_t(j) * kWave + lane;
      if (d < n_dwords) {
        const uint32_t e = ((wave * kWave) * 4u + uint32_t(j) * kWave + lane) * 4u;  // this group's place in the tile
        f32x4 r;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const bool first = e + uint32_t(k) < edge;
          r[k] = fmaf(first ? a0 : a1, float((w[j] >> (8 * k)) & 0xffu), first ? b0 : b1);
        }
        store_stream<NT>(&y4[d], r);
      }
    }
  } else {
  // the parameters of all four groups are requested before the first store (a streaming store is an ordering point
  // for the compiler: loads written after it are issued after it); a slot past the end takes the last group's
  uint32_t c4[4], sp4[4];
  float a4[4], b4[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint64_t d = wave_first + uint32_t(j) * kWave + lane;
    const uint32_t dc = (d < n_dwords) ? uint32_t(d) : (n_dwords != 0u ? n_dwords - 1u : 0u);
    uint32_t q;
    div_s.divmod(head + dc * 4u, q, sp4[j]);
    c4[j] = q - div_c.div(q) * C;
    a4[j] = scale[c4[j]];
    b4[j] = shift[c4[j]];
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint64_t d = wave_first + uint32_t(j) * kWave + lane;
    if (d < n_dwords) {
      uint32_t sp = sp4[j], c = c4[j];
      float a = a4[j], b = b4[j];
      f32x4 r;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        r[k] = fmaf(a, float((w[j] >> (8 * k)) & 0xffu), b);
        if (k < 3 && ++sp == S) {
          sp = 0;
          c = (c + 1 == C) ? 0 : c + 1;
          a = scale[c];
          b = shift[c];
        }
      }
      store_stream<NT>(&y4[d], r);
    }
  }
  }
  if (blockIdx.x == 0 && threadIdx.x < head + tail) {
    const uint32_t i = threadIdx.x < head ? threadIdx.x : n_dwords * 4u + threadIdx.x;
    const uint32_t q = div_s.div(i);
    const uint32_t c = q - div_c.div(q) * C;
    y_[i] = fmaf(scale[c], float(x_[i]), shift[c]);
  }
}

// ---------------------------------------------------------------------------
// per-channel sums and single-pass statistics
// ---------------------------------------------------------------------------

struct SumReduce {
  static constexpr int NIN = 1, NACC = 1;
  typedef Empty Param;
  float *y;
  bool square;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ void term(const Param &, float a, float, double &s0, double &, double &) const {
    const double d = double(a);
    s0 = square ? fma(d, d, s0) : s0 + d;
  }
  __device__ void finalize(uint32_t c, double s0, double, double) const { y[c] = float(s0); }
};

// mean and biased variance + eps in one pass over x.  Sums are taken about a
// per-channel shift K (the channel's first element), which keeps
// sum (x-K)^2 - (sum (x-K))^2 / n well conditioned for any offset of the data.
struct MeanVarReduce {
  static constexpr int NIN = 1, NACC = 2;
  typedef double Param;
  const float *x;
  float *mean, *var;
  uint32_t S;
  double n, eps;
  // running statistics updated in the same launch (null: none): y <- fma(rate, stat - y, y), the arithmetic of
  // online_average applied to the fp32 mean and variance that are stored
  float *run_mean = nullptr, *run_var = nullptr;
  float rate = 0.0f;
  __device__ Param load(uint32_t c) const { return double(x[size_t(c) * S]); }
  __device__ void term(const Param &k, float a, float, double &s0, double &s1, double &) const {
    const double d = double(a) - k;
    s0 += d;
    s1 = fma(d, d, s1);
  }
  __device__ void finalize(uint32_t c, double s0, double s1, double) const {
    const double k = n > 0.0 ? double(x[size_t(c) * S]) : 0.0;  // an empty array has no first element to read
    const float m = float(k + s0 / n);
    const float v = float((s1 - s0 * s0 / n) / n + eps);
    mean[c] = m;
    var[c] = v;
    if (run_mean) run_mean[c] = fmaf(rate, m - run_mean[c], run_mean[c]);
    if (run_var) run_var[c] = fmaf(rate, v - run_var[c], run_var[c]);
  }
};

// ---------------------------------------------------------------------------
// fused batch-norm forward maps
// ---------------------------------------------------------------------------

// y = relu_by_multiply((x - m) * rs): batch_norm followed by positive_clip in one pass
struct NormPositiveClipMap {
  const float *mean, *var;
  struct Param { float m, rs; };
  __device__ Param load(uint32_t c) const { return Param{mean[c], 1.0f / sqrtf(var[c])}; }
  __device__ float value(const Param &p, float x, float, uint32_t) const {
    const float t = (x - p.m) * p.rs;
    return t * float(t > 0.0f);
  }
  __device__ float accum(const Param &p, float x, float, uint32_t s, float old) const { return old + value(p, x, 0.0f, s); }
};

// y = fma((x - m) * rs, gamma[c], beta[c]): batch_norm followed by the per-channel affine
struct NormAffineMap {
  const float *mean, *var, *gamma, *beta;
  struct Param { float m, rs, g, b; };
  __device__ Param load(uint32_t c) const { return Param{mean[c], 1.0f / sqrtf(var[c]), gamma[c], beta[c]}; }
  __device__ float value(const Param &p, float x, float, uint32_t) const { return fmaf((x - p.m) * p.rs, p.g, p.b); }
  __device__ float accum(const Param &p, float x, float, uint32_t s, float old) const { return old + value(p, x, 0.0f, s); }
};

// ---------------------------------------------------------------------------
// fused batch-norm backward: one reduction pass over (dy, x), one map pass
// ---------------------------------------------------------------------------

// dvar = sum dy (x-m) * (-0.5 rs / v);  dmean = -rs sum dy + (sum (x-m)) (-2 dvar) / n.
// With a mask array (the ReLU output) dy is first multiplied by float(mask > 0).
template <bool MASKED>
struct NormBwdFusedReduce {
  static constexpr int NIN = MASKED ? 3 : 2, NACC = 3;  // a = dy, b = x, c = mask
  typedef double Param;
  const float *mean, *var;
  float *dmean, *dvar;
  double n;
  __device__ Param load(uint32_t c) const { return double(mean[c]); }
  __device__ void term(const Param &m, float dy, float x, double &s0, double &s1, double &s2) const {
    const double d = double(x) - m;
    s0 += double(dy);
    s1 = fma(double(dy), d, s1);
    s2 += d;
  }
  __device__ void term3(const Param &m, float dy, float x, float mask, double &s0, double &s1, double &s2) const {
    term(m, dy * float(mask > 0.0f), x, s0, s1, s2);
  }
  __device__ void finalize(uint32_t c, double s0, double s1, double s2) const {
    const double v = double(var[c]);
    const double rs = 1.0 / sqrt(v);
    const double dv = s1 * (-0.5 * rs / v);
    dvar[c] = float(dv);
    dmean[c] = float(-rs * s0 + s2 * (-2.0 * dv) / n);
  }
};

// dx (=|+=) dy*rs + dvar*(x-m)*2/n + dmean/n, each term in the arithmetic of the
// three separate launches it replaces and added in their order
template <bool MASKED>
struct NormBwdFusedMap {
  const float *mean, *var, *dmean, *dvar;
  float norm;
  struct Param { float m, rs, dv, dm; };
  __device__ Param load(uint32_t c) const {
    return Param{mean[c], 1.0f / sqrtf(var[c]), dvar[c], dmean[c] / norm};
  }
  __device__ float core(const Param &p, float dy, float x) const {
    return (dy * p.rs + p.dv * (x - p.m) * 2.0f / norm) + p.dm;
  }
  __device__ float value(const Param &p, float dy, float x, uint32_t) const { return core(p, dy, x); }
  __device__ float accum(const Param &p, float dy, float x, uint32_t, float old) const {
    return ((fmaf(dy, p.rs, old)) + p.dv * (x - p.m) * 2.0f / norm) + p.dm;
  }
  __device__ float value3(const Param &p, float dy, float x, float mask, uint32_t) const {
    return core(p, dy * float(mask > 0.0f), x);
  }
  __device__ float accum3(const Param &p, float dy, float x, float mask, uint32_t s, float old) const {
    return accum(p, dy * float(mask > 0.0f), x, s, old);
  }
};

// ---------------------------------------------------------------------------
// running average, arg-max
// ---------------------------------------------------------------------------

// y <- y + rate * (x - y)
struct OnlineAverageMap {
  float rate;
  __device__ float operator()(float x, float y) const { return fmaf(rate, x - y, y); }
};

__global__ __launch_bounds__(kBlock) void online_average_kernel(uint32_t len, float rate,
                                                                const float *__restrict__ x, float *y) {
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;  // 64-bit: index + stride can pass 2^32
  for (uint64_t i = uint64_t(blockIdx.x) * kBlock + threadIdx.x; i < len; i += stride) y[i] = fmaf(rate, x[i] - y[i], y[i]);
}

// First index of the strict maximum of each row of a [K (fastest), R] array;
// NaN never wins; a row without any value above -inf gives 0.  One wave per row.
// VEC: rows start on 16-byte boundaries (K a multiple of 4, x aligned), so a lane reads four consecutive classes.
template <bool VEC, int NT>
__global__ __launch_bounds__(kBlock) void arg_max_rows_kernel(uint32_t K, uint32_t R, const float *__restrict__ x,
                                                              uint32_t *__restrict__ out) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t wave = (blockIdx.x * kBlock + threadIdx.x) / kWave;
  const uint32_t n_waves = gridDim.x * (kBlock / kWave);
  for (uint64_t r = wave; r < R; r += n_waves) {
    const float *xr = x + size_t(r) * K;
    float top = -__builtin_huge_valf();
    uint32_t idx = 0xffffffffu;  // nothing above -inf seen yet
    if (VEC) {
      constexpr int U = 4;  // loads in flight per lane
      const f32x4 *xr4 = reinterpret_cast<const f32x4 *>(xr);
      const int32_t n4 = int32_t(K / 4u);
      // each step of the wave reads one 128-byte-aligned run of the array (for an array that starts on a line):
      // the groups are taken `a` places earlier than the row starts, and the first a lanes sit out the first step
      const int32_t a = int32_t((uint32_t(r) * (K / 4u)) & 7u);
      for (int32_t g0 = int32_t(lane) - a; g0 < n4; g0 += U * kWave) {
        f32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int32_t g = g0 + u * kWave;
          // a slot outside the row holds -inf, which never wins
          v[u] = (g >= 0 && g < n4) ? load_stream<NT>(&xr4[g]) : f32x4{-__builtin_huge_valf(), -__builtin_huge_valf(), -__builtin_huge_valf(), -__builtin_huge_valf()};
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {  // ascending class index inside the lane: the first maximum is kept
            if (v[u][j] > top) {
              top = v[u][j];
              idx = uint32_t(g0 + u * kWave) * 4u + uint32_t(j);
            }
          }
        }
      }
    } else {
#pragma unroll 4
      for (uint32_t k = lane; k < K; k += kWave) {
        const float v = xr[k];
        if (v > top) {
          top = v;
          idx = k;
        }
      }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      const float t2 = __shfl_xor(top, off, kWave);
      const uint32_t i2 = __shfl_xor(idx, off, kWave);
      if (t2 > top || (t2 == top && i2 < idx)) {
        top = t2;
        idx = i2;
      }
    }
    if (lane == 0) out[r] = (idx == 0xffffffffu) ? 0u : idx;
  }
}

void launch_quantize(const char *symbol, uint32_t len, float lo, float hi, const float *x, uint8_t *y,
                     CUstream_st *stream) {
  if (len == 0) return;
  const float scale = (hi - lo) / 255.0f;
  hipStream_t s = as_stream(stream);
  uint32_t head = uint32_t((128u - (reinterpret_cast<uintptr_t>(y) & 127u)) & 127u);  // bytes = elements of y
  if (head > len) head = len;
  const uint32_t groups = (len - head) / 4, tail = (len - head) % 4;
  const uint32_t blocks = (groups + kBlock * 4 - 1) / (kBlock * 4);
  quantize_u8x16_kernel<<<blocks ? blocks : 1, kBlock, 0, s>>>(head, groups, tail, lo, scale, x, y);
  note_launch(symbol);
}

}  // namespace
}  // namespace anode

using namespace anode;

ANODE_EXPORT void anode_gpu_quantize_u8_packed_f32(uint32_t len, float lo, float hi, const float *x, uint8_t *y,
                                                   const KernelConfig *, CUstream_st *stream) {
  launch_quantize(__func__, len, lo, hi, x, y, stream);
}

ANODE_EXPORT void anode_gpu_bcast_flat_mult_I1b_I2ab_Oab_packed_f32(uint32_t inner_dim, uint32_t bcast_dim,
                                                                    const float *lx, const float *rx, float *y,
                                                                    const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, false>(__func__, inner_dim, bcast_dim, 1, BcastMultMap{lx}, rx, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_bcast_flat_mult_add_I1b_I2ab_Oab_packed_f32(uint32_t inner_dim, uint32_t bcast_dim,
                                                                        const float *lx, const float *rx,
                                                                        const float *shift, float *y,
                                                                        const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, false>(__func__, inner_dim, bcast_dim, 1, BcastMultAddMap{lx, shift}, rx, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_bcast_flat_mult_I1b_I2abc_Oabc_packed_f32(uint32_t inner_dim, uint32_t bcast_dim,
                                                                      uint32_t outer_dim, const float *lx,
                                                                      const float *rx, float *y,
                                                                      const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, false>(__func__, inner_dim, bcast_dim, outer_dim, BcastMultMap{lx}, rx, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_bcast_flat_mult_add_I1b_I2abc_Oabc_packed_f32(uint32_t inner_dim, uint32_t bcast_dim,
                                                                          uint32_t outer_dim, const float *lx,
                                                                          const float *rx, const float *shift,
                                                                          float *y, const KernelConfig *,
                                                                          CUstream_st *stream) {
  launch_chan_map<1, false>(__func__, inner_dim, bcast_dim, outer_dim, BcastMultAddMap{lx, shift}, rx, nullptr, y,
                            stream);
}

ANODE_EXPORT void anode_gpu_flat_mult_f32(uint32_t len, const float *lx, const float *rx, float *y,
                                          const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<2, false>(__func__, len, 1, 1, FlatMultMap{}, lx, rx, y, stream);
}

ANODE_EXPORT void anode_gpu_flat_mult_add_f32(uint32_t len, const float *lx, const float *rx, const float *shift,
                                              float *y, const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<3, false>(__func__, len, 1, 1, FlatMultAddMap{}, lx, rx, y, stream, shift);
}

ANODE_EXPORT void anode_gpu_bcast_dequantize_u8_I1b_I2abc_Oabc_packed_f32(uint32_t inner_dim, uint32_t bcast_dim,
                                                                          uint32_t outer_dim, const float *scale,
                                                                          const float *shift, const uint8_t *x,
                                                                          float *y, const KernelConfig *,
                                                                          CUstream_st *stream) {
  const uint32_t len = checked_len(inner_dim, bcast_dim, outer_dim, __func__);
  if (len == 0) return;
  hipStream_t s = as_stream(stream);
  const FastDiv div_s(inner_dim), div_c(bcast_dim);
  const uint32_t head = head_to_align_line(y, len);
  const uint32_t dwords = (len - head) / 4, tail = (len - head) % 4;
  const uint32_t blocks = (dwords + kBlock * 4 - 1) / (kBlock * 4);
  with_stream_policy(stream_policy(size_t(len) * sizeof(float), tuning().nontemporal) & kNtStore, [&](auto policy) {
    if (inner_dim >= uint32_t(kBlock * 16)) {
      bcast_dequantize_u8x16_kernel<decltype(policy)::value, true>
          <<<blocks ? blocks : 1, kBlock, 0, s>>>(head, dwords, tail, div_s, div_c, scale, shift, x, y);
    } else {
      bcast_dequantize_u8x16_kernel<decltype(policy)::value, false>
          <<<blocks ? blocks : 1, kBlock, 0, s>>>(head, dwords, tail, div_s, div_c, scale, shift, x, y);
    }
  });
  note_launch(__func__);
}

ANODE_EXPORT void anode_gpu_sum_Iab_Ob_packed_deterministic_f32(uint32_t reduce_dim, uint32_t outer_dim,
                                                                const float *x, float *y, const KernelConfig *,
                                                                CUstream_st *stream) {
  launch_chan_reduce(__func__, reduce_dim, outer_dim, 1, SumReduce{y, false}, x, nullptr, stream);
}

ANODE_EXPORT void anode_gpu_sum_Iabc_Ob_packed_deterministic_f32(uint32_t reduce_inner_dim, uint32_t mid_dim,
                                                                 uint32_t reduce_outer_dim, const float *x, float *y,
                                                                 const KernelConfig *, CUstream_st *stream) {
  launch_chan_reduce(__func__, reduce_inner_dim, mid_dim, reduce_outer_dim, SumReduce{y, false}, x, nullptr, stream);
}

ANODE_EXPORT void anode_gpu_square_sum_Iabc_Ob_packed_deterministic_f32(uint32_t reduce_inner_dim, uint32_t mid_dim,
                                                                        uint32_t reduce_outer_dim, const float *x,
                                                                        float *y, const KernelConfig *,
                                                                        CUstream_st *stream) {
  launch_chan_reduce(__func__, reduce_inner_dim, mid_dim, reduce_outer_dim, SumReduce{y, true}, x, nullptr, stream);
}

ANODE_EXPORT void anode_gpu_batch_mean_var_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, float epsilon,
                                                          const float *x, float *mean, float *var,
                                                          const KernelConfig *, CUstream_st *stream) {
  launch_chan_reduce(__func__, dim0, dim1, dim2,
                     MeanVarReduce{x, mean, var, dim0, double(dim0) * double(dim2), double(epsilon)}, x, nullptr, stream);
}

// The same with the layer's running statistics updated by the workgroup that finalises a channel: what
// src/ops.rs:999-1003 does with batch_mean, batch_var and two online_average launches.
ANODE_EXPORT void anode_gpu_batch_mean_var_online_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                                 float epsilon, float rate, const float *x,
                                                                 float *mean, float *var, float *run_mean,
                                                                 float *run_var, const KernelConfig *,
                                                                 CUstream_st *stream) {
  MeanVarReduce op{x, mean, var, dim0, double(dim0) * double(dim2), double(epsilon)};
  op.run_mean = run_mean;
  op.run_var = run_var;
  op.rate = rate;
  launch_chan_reduce(__func__, dim0, dim1, dim2, op, x, nullptr, stream);
}

// ---------------------------------------------------------------------------
// batch_mean_var for callers that cannot allocate (code under HIP graph
// capture, serving loops, harnesses that forbid hipMalloc): the partial sums
// live in a device array that is part of the library's image, one copy per GPU.
// ---------------------------------------------------------------------------
namespace {
constexpr size_t kNoAllocScratchBytes = size_t(4) << 20;  // 4 MiB per GPU, held until the process ends
constexpr int kNoAllocMaxDevices = 64;
std::mutex g_noalloc_mutex;
void *g_noalloc_ptr[kNoAllocMaxDevices] = {};  // device address of `scratch` on each GPU, looked up once
// Calls on different streams of one GPU share that GPU's array.  Outside graph capture they are put in order on the
// device: every call records this event behind its kernels, and a call on another stream than the last one waits for
// it first.  The event is created with the address look-up, once per device; the mutex is held from the wait to the
// record, so host threads cannot interleave their calls.
std::mutex g_noalloc_order_mutex;
hipEvent_t g_noalloc_done[kNoAllocMaxDevices] = {};
hipStream_t g_noalloc_last_stream[kNoAllocMaxDevices] = {};
bool g_noalloc_recorded[kNoAllocMaxDevices] = {};
}  // namespace

static __device__ __align__(256) double scratch[kNoAllocScratchBytes / sizeof(double)];

// The device address of this GPU's copy of `scratch` (in host code the array's name is only a handle for the
// symbol, not an address a kernel could use).  Looked up on the first call with each device current.
static void *noalloc_scratch_of_current_device(const char *symbol) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kNoAllocMaxDevices) {
    note_error(symbol, hipErrorInvalidDevice, "no current device to take the scratch array from");
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_noalloc_mutex);
  if (!g_noalloc_ptr[dev]) {
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      note_error(symbol, e != hipSuccess ? e : hipErrorInvalidSymbol, "cannot look up the scratch array");
      return nullptr;
    }
    hipEvent_t done = nullptr;
    const hipError_t ee = hipEventCreateWithFlags(&done, hipEventDisableTiming);
    if (ee != hipSuccess || !done) {
      note_error(symbol, ee != hipSuccess ? ee : hipErrorUnknown, "cannot create the event that orders calls on the scratch array");
      return nullptr;
    }
    g_noalloc_done[dev] = done;
    g_noalloc_ptr[dev] = p;
  }
  return g_noalloc_ptr[dev];
}

ANODE_EXPORT int anode_gpu_batch_mean_var_3d1_packed_noalloc_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                                 float epsilon, const float *x, float *mean,
                                                                 float *var, const KernelConfig *,
                                                                 CUstream_st *stream) {
  // Sizes are checked before anything touches the device, so that a refusal has no side effect; the element count
  // first, as in every other entry point (the tiling below is not planned for counts that do not fit 32 bits).
  (void)checked_len(dim0, dim1, dim2, __func__);
  const bool ptrs_aligned = true;  // (16-byte loads from any 4-byte aligned address, as in launch_chan_reduce)
  const ReducePlan pl = plan_chan_reduce(dim0, dim1, dim2, ptrs_aligned, uint32_t(tuning().reduce_wg_target),
                                         MeanVarReduce::NIN);
  const size_t need = chan_reduce_scratch_bytes(pl, MeanVarReduce::NACC);
  if (need > kNoAllocScratchBytes) {
    std::fprintf(stderr,
                 "%s: [%u, %u, %u] needs %zu bytes of partial sums, more than the %zu bytes of the static scratch "
                 "array; use anode_gpu_batch_mean_var_3d1_packed_f32; nothing was enqueued\n",
                 __func__, dim0, dim1, dim2, need, kNoAllocScratchBytes);
    return kReduceScratchTooSmall;
  }
  FixedScratch fixed{nullptr, kNoAllocScratchBytes};
  const MeanVarReduce op{x, mean, var, dim0, double(dim0) * double(dim2), double(epsilon)};
  if (need == 0) return launch_chan_reduce(__func__, dim0, dim1, dim2, op, x, nullptr, stream, nullptr, &fixed);
  fixed.ptr = noalloc_scratch_of_current_device(__func__);
  if (!fixed.ptr) return kReduceScratchUnavailable;
  int dev = 0;
  (void)hipGetDevice(&dev);  // (checked by the look-up above)
  hipStream_t s = as_stream(stream);
  std::lock_guard<std::mutex> order(g_noalloc_order_mutex);
  // A stream under capture takes no part in the ordering: an event recorded into a capture cannot be waited for
  // from outside it, and a captured call runs whenever its graph is launched.  Such callers keep their calls on one
  // GPU from overlapping themselves.  (A capture state that cannot be read counts as capturing.)
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  const bool plain = hipStreamIsCapturing(s, &capturing) == hipSuccess && capturing == hipStreamCaptureStatusNone;
  if (!plain) (void)hipGetLastError();
  if (plain && g_noalloc_recorded[dev] && g_noalloc_last_stream[dev] != s) {
    const hipError_t w = hipStreamWaitEvent(s, g_noalloc_done[dev], 0);
    if (w != hipSuccess) {
      note_error(__func__, w, "cannot wait for the previous call on the scratch array; nothing was enqueued");
      return kReduceScratchUnavailable;
    }
  }
  // Every partial that the second kernel reads is written by the first kernel of the same call, so nothing in
  // the array has to start at zero.
  const int rc = launch_chan_reduce(__func__, dim0, dim1, dim2, op, x, nullptr, stream, nullptr, &fixed);
  if (plain) {
    const hipError_t r = hipEventRecord(g_noalloc_done[dev], s);
    if (r == hipSuccess) {
      g_noalloc_last_stream[dev] = s;
      g_noalloc_recorded[dev] = true;
    } else {
      note_error(__func__, r, "cannot record the event that orders calls on the scratch array");
    }
  }
  return rc;
}

ANODE_EXPORT void anode_gpu_batch_norm_positive_clip_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                                    const float *x, const float *mean,
                                                                    const float *var, float *y, const KernelConfig *,
                                                                    CUstream_st *stream) {
  launch_chan_map<1, false>(__func__, dim0, dim1, dim2, NormPositiveClipMap{mean, var}, x, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_affine_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                             const float *x, const float *mean, const float *var,
                                                             const float *gamma, const float *beta, float *y,
                                                             const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, false>(__func__, dim0, dim1, dim2, NormAffineMap{mean, var, gamma, beta}, x, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_bwd_reduce_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                                 const float *dy, const float *x, const float *mean,
                                                                 const float *var, const float *mask, float *dmean,
                                                                 float *dvar, const KernelConfig *,
                                                                 CUstream_st *stream) {
  const double n = double(dim0) * double(dim2);
  if (mask) {
    launch_chan_reduce(__func__, dim0, dim1, dim2, NormBwdFusedReduce<true>{mean, var, dmean, dvar, n}, dy, x, stream, mask);
  } else {
    launch_chan_reduce(__func__, dim0, dim1, dim2, NormBwdFusedReduce<false>{mean, var, dmean, dvar, n}, dy, x, stream);
  }
}

static void bwd_apply(const char *symbol, bool accumulate, uint32_t dim0, uint32_t dim1, uint32_t dim2,
                      const float *dy, const float *x, const float *mean, const float *var, const float *dmean,
                      const float *dvar, const float *mask, float *dx, CUstream_st *stream) {
  const float norm = float(dim0) * float(dim2);
  if (mask) {
    const NormBwdFusedMap<true> op{mean, var, dmean, dvar, norm};
    if (accumulate) {
      launch_chan_map<3, true>(symbol, dim0, dim1, dim2, op, dy, x, dx, stream, mask);
    } else {
      launch_chan_map<3, false>(symbol, dim0, dim1, dim2, op, dy, x, dx, stream, mask);
    }
  } else {
    const NormBwdFusedMap<false> op{mean, var, dmean, dvar, norm};
    if (accumulate) {
      launch_chan_map<2, true>(symbol, dim0, dim1, dim2, op, dy, x, dx, stream);
    } else {
      launch_chan_map<2, false>(symbol, dim0, dim1, dim2, op, dy, x, dx, stream);
    }
  }
}

ANODE_EXPORT void anode_gpu_batch_norm_bwd_apply_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                                const float *dy, const float *x, const float *mean,
                                                                const float *var, const float *dmean,
                                                                const float *dvar, const float *mask, float *dx,
                                                                const KernelConfig *, CUstream_st *stream) {
  bwd_apply(__func__, false, dim0, dim1, dim2, dy, x, mean, var, dmean, dvar, mask, dx, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_bwd_apply_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1,
                                                                           uint32_t dim2, const float *dy,
                                                                           const float *x, const float *mean,
                                                                           const float *var, const float *dmean,
                                                                           const float *dvar, const float *mask,
                                                                           float *dx, const KernelConfig *,
                                                                           CUstream_st *stream) {
  bwd_apply(__func__, true, dim0, dim1, dim2, dy, x, mean, var, dmean, dvar, mask, dx, stream);
}

ANODE_EXPORT void anode_gpu_online_average_packed_f32(uint32_t len, float rate, const float *x, float *y,
                                                      const KernelConfig *, CUstream_st *stream) {
  if (len == 0) return;
  online_average_kernel<<<stream_grid(len, 1), kBlock, 0, as_stream(stream)>>>(len, rate, x, y);
  note_launch(__func__);
}

ANODE_EXPORT void anode_gpu_arg_max_packed_u32(uint32_t dim0, uint32_t dim1, const float *x, uint32_t *index,
                                               const KernelConfig *, CUstream_st *stream) {
  (void)checked_len(dim0, dim1, 1, __func__);
  if (dim1 == 0) return;
  const uint32_t waves_per_block = kBlock / kWave;
  uint32_t blocks = (dim1 + waves_per_block - 1) / waves_per_block;
  const uint32_t cap = 1u << 24;  // one row per wave; the kernel loops only beyond that
  if (blocks > cap) blocks = cap;
  if (dim0 % 4u == 0) {  // (16-byte loads from any 4-byte aligned address)
    const int nt = stream_policy(size_t(dim0) * dim1 * sizeof(float), tuning().reduce_nontemporal) & kNtLoad;
    if (nt) {
      arg_max_rows_kernel<true, kNtLoad><<<blocks, kBlock, 0, as_stream(stream)>>>(dim0, dim1, x, index);
    } else {
      arg_max_rows_kernel<true, 0><<<blocks, kBlock, 0, as_stream(stream)>>>(dim0, dim1, x, index);
    }
  } else {
    arg_max_rows_kernel<false, 0><<<blocks, kBlock, 0, as_stream(stream)>>>(dim0, dim1, x, index);
  }
  note_launch(__func__);
}

// The host rule of src/utils/mod.rs:31-41, for callers that keep logits on the host.
ANODE_EXPORT size_t anode_host_arg_max_f32(const float *xs, size_t len) {
  float top_x = -__builtin_huge_valf();
  size_t top_k = 0;
  for (size_t k = 0; k < len; ++k) {
    if (xs[k] > top_x) {
      top_x = xs[k];
      top_k = k;
    }
  }
  return top_k;
}
