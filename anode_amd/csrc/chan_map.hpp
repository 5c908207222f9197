// Elementwise maps over a packed [S, C, N] array (S fastest) whose arithmetic
// depends on the element's channel c: out[s,c,n] = f(param[c], a[s,c,n], b[s,c,n]).
//
// The array is walked as a flat sequence of 16-byte groups, exactly like the
// channel-free maps; the channel of a group's first element comes from two
// multiply-high divisions by launch-invariant divisors (no hardware divide per
// element), and the (s, c) pair is then advanced incrementally inside the
// group, reloading the per-channel parameters only when a channel boundary is
// crossed.  This keeps full 16-byte accesses for every S, including S that is
// not a multiple of 4 (7x7 feature maps) and S == 1, and for arrays that start
// at any element (a head of up to 31 elements is peeled so that the stores
// start on a 128-byte line; the inputs are read where they lie).
#pragma once

#include "common.hpp"

namespace anode {

// Op concept:
//   struct Param;                                  per-channel values
//   __device__ Param load(uint32_t c) const;
//   __device__ float value(const Param&, float a, float b, uint32_t s) const;
//   __device__ float accum(const Param&, float a, float b, uint32_t s, float old) const;
// where s is the element's position inside its channel run.  Ops with a third
// element input (NIN == 3) define value3/accum3 taking (a, b, c) instead.
template <typename V> struct VecLanes;
template <> struct VecLanes<float> { static constexpr int n = 1; };
template <> struct VecLanes<f32x4> { static constexpr int n = 4; };

template <typename V>
__device__ inline float lane_get(const V &v, int k);
template <>
__device__ inline float lane_get<float>(const float &v, int) { return v; }
template <>
__device__ inline float lane_get<f32x4>(const f32x4 &v, int k) { return v[k]; }

template <typename V>
__device__ inline void lane_set(V &v, int k, float x);
template <>
__device__ inline void lane_set<float>(float &v, int, float x) { v = x; }
template <>
__device__ inline void lane_set<f32x4>(f32x4 &v, int k, float x) { v[k] = x; }

template <int NIN, bool ACC, typename Op, typename P>
__device__ inline float chan_map_apply(const Op &op, const P &p, float x, float y, float z, uint32_t s, float old) {
  if constexpr (NIN >= 3) {
    return ACC ? op.accum3(p, x, y, z, s, old) : op.value3(p, x, y, z, s);
  } else {
    return ACC ? op.accum(p, x, y, s, old) : op.value(p, x, y, s);
  }
}

// PAIR selects how a group that crosses a channel boundary gets its second parameter set: fetched up front beside
// the first (channels of a few dozen elements, where a quarter of the groups cross), or on demand while walking
// the group (long channels, where almost none does and the extra fetch and selects only cost issue slots).
// `head` single elements (0 to 31) come before the groups, `tail` after them, both handled by workgroup 0: the
// host picks head so that the groups of `out_` start on a 128-byte line wherever the array lies; the inputs are
// read where they lie (4-byte aligned 16-byte loads).
template <int NIN, bool ACC, int NT, bool PAIR, typename Op>
__global__ __launch_bounds__(kBlock) void chan_map_kernel(uint32_t head, uint32_t n_groups, uint32_t tail,
                                                          FastDiv div_s, FastDiv div_c, Op op, const float *a_,
                                                          const float *b_, const float *c_, float *out_) {
  typedef f32x4 V;
  constexpr int L = 4;
  const V *a = reinterpret_cast<const V *>(a_ + head);
  const V *b = reinterpret_cast<const V *>(b_ + head);
  const V *c3 = reinterpret_cast<const V *>(c_ + head);
  V *out = reinterpret_cast<V *>(out_ + head);
  const uint32_t S = div_s.d, C = div_c.d;
  // one group per thread on a full grid; the loop only runs more than once under the grid cap of the tuning hook
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;  // 64-bit: index + stride can pass 2^32
  for (uint64_t g = uint64_t(blockIdx.x) * kBlock + threadIdx.x; g < n_groups; g += stride) {
    V va, vb, vc, vo;
    if (NIN >= 1) va = load_stream<NT>(&a[g]);
    if (NIN >= 2) vb = load_stream<NT>(&b[g]);
    if (NIN >= 3) vc = load_stream<NT>(&c3[g]);
    if (ACC) vo = load_stream<NT>(&out[g]);
    uint32_t q, s;
    div_s.divmod(head + uint32_t(g) * uint32_t(L), q, s);
    uint32_t c = q - div_c.div(q) * C;
    V r;
    if (PAIR) {  // the host guarantees S >= L here
      // A group spans at most two channels.  Both parameter sets are fetched up front, next to the element
      // loads, so that a group that crosses a channel boundary does not wait for a second, dependent fetch
      // (with S = 49 a quarter of the groups cross).
      const uint32_t room = S - s;  // elements of the group that still belong to channel c
      const typename Op::Param p0 = op.load(c);
      const uint32_t c1 = (c + 1 == C) ? 0 : c + 1;
      // (fetched without a branch, from channel c again where the group does not cross: a branch round the
      // fetch would make it wait for the loads issued before it)
      const typename Op::Param p1 = op.load(room < uint32_t(L) ? c1 : c);
#pragma unroll
      for (int k = 0; k < L; ++k) {
        const bool first = uint32_t(k) < room;
        const float x = (NIN >= 1) ? va[k] : 0.0f;
        const float y = (NIN >= 2) ? vb[k] : 0.0f;
        const float z = (NIN >= 3) ? vc[k] : 0.0f;
        const float old = ACC ? vo[k] : 0.0f;
        const typename Op::Param pk = first ? p0 : p1;
        const uint32_t sk = first ? s + uint32_t(k) : uint32_t(k) - room;
        r[k] = chan_map_apply<NIN, ACC>(op, pk, x, y, z, sk, old);
      }
    } else {
      // channels shorter than a group: walk (s, c) element by element
      typename Op::Param p = op.load(c);
#pragma unroll
      for (int k = 0; k < L; ++k) {
        const float x = (NIN >= 1) ? va[k] : 0.0f;
        const float y = (NIN >= 2) ? vb[k] : 0.0f;
        const float z = (NIN >= 3) ? vc[k] : 0.0f;
        r[k] = chan_map_apply<NIN, ACC>(op, p, x, y, z, s, ACC ? vo[k] : 0.0f);
        if (k + 1 < L) {
          if (++s == S) {
            s = 0;
            c = (c + 1 == C) ? 0 : c + 1;
            p = op.load(c);
          }
        }
      }
    }
    store_stream<NT>(&out[g], r);
  }
  if (blockIdx.x == 0 && threadIdx.x < head + tail) {
    const uint32_t i = threadIdx.x < head ? threadIdx.x : n_groups * uint32_t(L) + threadIdx.x;
    uint32_t q, s;
    div_s.divmod(i, q, s);
    const uint32_t c = q - div_c.div(q) * C;
    const typename Op::Param p = op.load(c);
    const float x = (NIN >= 1) ? a_[i] : 0.0f;
    const float y = (NIN >= 2) ? b_[i] : 0.0f;
    const float z = (NIN >= 3) ? c_[i] : 0.0f;
    out_[i] = chan_map_apply<NIN, ACC>(op, p, x, y, z, s, ACC ? out_[i] : 0.0f);
  }
}

// One element per channel and sample (S = 1: batch-norm over a [C, N] matrix): a 16-byte group then spans four
// channels, and walking it element by element fetches and prepares (a division and a square root for batch-norm)
// one parameter set per ELEMENT.  Here a thread keeps one group position of the C-float sample period, prepares its
// four parameter sets once, and walks kColSamples samples at that position, eight 16-byte loads in flight per
// input.  Needs C a multiple of 4 and aligned arrays.  (Written for any S < 4, but with two or three elements per
// channel the flat walk is as fast or faster: batch_var_bwd_accumulate at [2, 512, 65536] 6.5 TB/s against 5.7.)
constexpr uint32_t kColSamples = 16;

template <int NIN, bool ACC, int NT, typename Op>
__global__ __launch_bounds__(kBlock) void chan_map_cols_kernel(uint32_t S, uint32_t N, uint32_t total_threads,
                                                               FastDiv div_gpp, FastDiv div_s, Op op,
                                                               const float *a_, const float *b_, const float *c_,
                                                               float *out_) {
  constexpr int B = 8;  // samples requested together
  const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
  if (t >= total_threads) return;
  const uint32_t gpp = div_gpp.d;  // groups per sample period
  uint32_t chunk, g;
  div_gpp.divmod(t, chunk, g);
  typename Op::Param prm[4];
  uint32_t pos[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    uint32_t c;
    div_s.divmod(g * 4u + uint32_t(k), c, pos[k]);
    prm[k] = op.load(c);
  }
  const size_t period4 = size_t(gpp);  // 16-byte groups per sample
  const f32x4 *a = reinterpret_cast<const f32x4 *>(a_);
  const f32x4 *b = reinterpret_cast<const f32x4 *>(b_);
  const f32x4 *c3 = reinterpret_cast<const f32x4 *>(c_);
  f32x4 *out = reinterpret_cast<f32x4 *>(out_);
  const uint32_t n0 = chunk * kColSamples;
  const uint32_t n1 = (N - n0 < kColSamples) ? N : n0 + kColSamples;
  for (uint32_t nb = n0; nb < n1; nb += uint32_t(B)) {
    f32x4 va[B], vb[B], vc[B], vo[B];
#pragma unroll
    for (int u = 0; u < B; ++u) {  // unconditional: a slot past the chunk's end reads its last sample again
      const uint32_t n = nb + uint32_t(u) < n1 ? nb + uint32_t(u) : n1 - 1u;
      const size_t at = size_t(n) * period4 + g;
      if (NIN >= 1) va[u] = load_stream<NT>(&a[at]);
      if (NIN >= 2) vb[u] = load_stream<NT>(&b[at]);
      if (NIN >= 3) vc[u] = load_stream<NT>(&c3[at]);
      if (ACC) vo[u] = load_stream<NT>(&out[at]);
    }
#pragma unroll
    for (int u = 0; u < B; ++u) {
      if (nb + uint32_t(u) < n1) {
        f32x4 r;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float x = (NIN >= 1) ? va[u][k] : 0.0f;
          const float y = (NIN >= 2) ? vb[u][k] : 0.0f;
          const float z = (NIN >= 3) ? vc[u][k] : 0.0f;
          r[k] = chan_map_apply<NIN, ACC>(op, prm[k], x, y, z, pos[k], ACC ? vo[u][k] : 0.0f);
        }
        store_stream<NT>(&out[size_t(nb + uint32_t(u)) * period4 + g], r);
      }
    }
  }
}

// a, b may be null when NIN says they are unused.
template <int NIN, bool ACC, typename Op>
void launch_chan_map(const char *symbol, uint32_t S, uint32_t C, uint32_t N, Op op, const float *a,
                     const float *b, float *out, CUstream_st *stream, const float *c = nullptr) {
  const uint32_t len = checked_len(S, C, N, symbol);
  if (len == 0) return;
  const Tuning &t = tuning();
  hipStream_t s = as_stream(stream);
  const FastDiv div_s(S), div_c(C);
  const bool vec = aligned16(out) && (NIN < 1 || aligned16(a)) && (NIN < 2 || aligned16(b)) &&
                   (NIN < 3 || aligned16(c));
  const int nt = stream_policy(size_t(len) * sizeof(float), t.nontemporal);
  if (vec && S == 1 && C % 4 == 0 && C >= 64 && N >= kColSamples) {  // (fewer channels: a wave's loads would scatter)
    const uint32_t gpp = uint32_t(uint64_t(C) * S / 4);
    const uint64_t threads = uint64_t(gpp) * ((N + kColSamples - 1) / kColSamples);  // <= len / 4
    const FastDiv div_gpp(gpp);
    with_stream_policy(nt, [&](auto policy) {
      constexpr int NT = decltype(policy)::value;
      chan_map_cols_kernel<NIN, ACC, NT, Op><<<uint32_t((threads + kBlock - 1) / kBlock), kBlock, 0, s>>>(
          S, N, uint32_t(threads), div_gpp, div_s, op, a, b, c, out);
    });
  } else {
    const uint32_t head = head_to_align_line(out, len);
    const uint32_t groups = (len - head) / 4, tail = (len - head) % 4;
    const bool pair = S >= 4 && S < 4096;
    with_stream_policy(nt, [&](auto policy) {
      constexpr int NT = decltype(policy)::value;
      if (pair) {
        chan_map_kernel<NIN, ACC, NT, true, Op>
            <<<stream_grid(groups ? groups : 1, 1), kBlock, 0, s>>>(head, groups, tail, div_s, div_c, op, a, b, c, out);
      } else {
        chan_map_kernel<NIN, ACC, NT, false, Op>
            <<<stream_grid(groups ? groups : 1, 1), kBlock, 0, s>>>(head, groups, tail, div_s, div_c, op, a, b, c, out);
      }
    });
  }
  note_launch(symbol);
}

}  // namespace anode
