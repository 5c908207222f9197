// Softmax with the categorical negative log-likelihood gather and its backward.
//
// Row form  [K classes (fastest), R rows]: the reduced axis is contiguous.
//   K <= 32     : one thread per row; a workgroup's 256 rows are staged through LDS with coalesced accesses;
//   K <= 64     : a row lives in a group of 64 lanes;
//   K <= 2048   : one wave per row, the row held in registers (lane l owns k = l, l+64, ...);
//   K <= 16384  : one workgroup per row, the row held in registers;
//   larger K    : one workgroup per row, online max/sum pass then a normalising pass.
// N-d form  [P pixels (fastest), C classes, N]: the reduced axis has stride P.
//   One thread owns 4 consecutive pixels (16-byte accesses, coalesced across the
//   wave), holds the C values of its pixels in registers and so reads x once.
// Every reduction order is fixed by the geometry, so results are reproducible.
// The block and the deterministic entry points of the reference share one
// implementation here and accept any K.
#include "chan_map.hpp"
#include "common.hpp"

#include <cmath>
#include <cstring>

namespace anode {
namespace {

constexpr float kNegInf = -__builtin_huge_valf();

// ---------------------------------------------------------------------------
// row softmax
// ---------------------------------------------------------------------------

// Optional fused label gather, and optional fused backward, of the row kernels (cat == nullptr: none).  The thread
// that has just stored probability p of class k also writes what the separate kernels would compute from the stored
// value: nll = -log(p) if k is the row's label (a label >= K gives NaN, or 0 with `ignore`, written by the thread
// that holds class 0), and, when dy is given, dx[k] = dy[row] * (p - float(label == k)) (softmax.cu:188-193).
struct RowNll {
  const uint32_t *cat;
  float *nll;
  bool ignore;
  const float *dy;  // with dx: the upstream gradient per row, known before the forward pass (e.g. ones for a summed loss)
  float *dx;
  __device__ bool on() const { return cat != nullptr; }
  __device__ uint32_t label(uint64_t r) const { return cat[r]; }
  // called by the thread that holds class k of row r, with the stored probability
  __device__ void emit_nll(uint64_t r, uint32_t K, uint32_t label, uint32_t k, float prob) const {
    if (k == label) {
      nll[r] = -logf(prob);
    } else if (k == 0 && label >= K) {
      nll[r] = ignore ? 0.0f : __builtin_nanf("");
    }
  }
  // softmax.cu:177-225: the gradient of class k for upstream gradient dyr
  __device__ static float grad(float dyr, uint32_t label, uint32_t k, float prob) {
    return dyr * (prob - float(label == k));
  }
  // the same, and the gradient stored element by element (kernels whose lanes hold consecutive classes)
  __device__ void emit(uint64_t r, uint32_t K, uint32_t label, uint32_t k, float prob) const {
    emit_nll(r, K, label, k, prob);
    if (dx != nullptr) dx[size_t(r) * K + k] = grad(dy[r], label, k, prob);
  }
};

// max(a, b) as the single hardware instruction: a NaN operand yields the other operand and a signalling NaN is
// quieted, which is fmaxf(); the library call costs two more instructions per element to canonicalise its inputs.
__device__ inline float max1(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ inline float vmax(float a, float b) { return max1(a, b); }
__device__ inline f32x4 vmax(f32x4 a, f32x4 b) {
  return f32x4{max1(a.x, b.x), max1(a.y, b.y), max1(a.z, b.z), max1(a.w, b.w)};
}

// exp(d) for d <= 0 (the difference to a row's maximum): 2^(d * log2 e) with the hardware exponential, corrected
// for the rounding of the product, r = fma(d, log2 e, -t), by the factor 1 + r ln 2.  Seven instructions instead of
// the sixteen of expf(), which the softmax kernels feel: 76 exponentials per thread made the n-d kernel 40 % VALU-busy.
// Relative error <= 3e-7 (+ 2e-8 |d| from the rounding of log2 e) while the result is a normal number; below
// 2^-126 the hardware exponential returns 0, far under any probability that is compared (sums start at exp(0) = 1).
// d = -inf gives 0 (the residual, inf - inf, is clamped before use), NaN gives NaN.
__device__ inline float exp_nonpos(float d) {
  constexpr float kLog2e = 1.44269502f, kLn2 = 0.693147182f;
  const float t = d * kLog2e;
  const float r = __builtin_amdgcn_fmed3f(fmaf(d, kLog2e, -t), -1.0f, 1.0f);
  const float e = __builtin_amdgcn_exp2f(t);
  return fmaf(e, r * kLn2, e);
}
__device__ inline f32x4 vexp4(f32x4 a) { return f32x4{exp_nonpos(a.x), exp_nonpos(a.y), exp_nonpos(a.z), exp_nonpos(a.w)}; }
// Marks the point from which a loaded value is known to have arrived.  The streaming stores are inline assembly,
// which the compiler's wait-count bookkeeping does not see: where the first use of an earlier load sits in a
// conditional block after such stores, the wait it inserts there (for "the load") also waits for every store
// issued since, one store at a time.  Using the value once before the stores begin removes those waits.
// (The memory clobber keeps the loads written before the mark before it, and those after it after it.)
__device__ inline void arrived(float v) { asm volatile("" ::"v"(v) : "memory"); }
__device__ inline void arrived(uint32_t v) { asm volatile("" ::"v"(v) : "memory"); }
__device__ inline void arrived(f32x4 v) { asm volatile("" ::"v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w) : "memory"); }
__device__ inline void arrived(u32x4 v) { asm volatile("" ::"v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w) : "memory"); }
__device__ inline void issue_order_fence() { asm volatile("" ::: "memory"); }

// K <= 32 * G: G = 1, 2, 4 or 8 lanes per row, up to KMAX <= 32 values per lane.  A workgroup takes 256 / G
// consecutive rows, which are contiguous floats: they are copied to LDS as they lie in memory, 16 bytes per lane,
// each lane group normalises its row in registers, and the tile goes back the same way, so every global access
// is a full-width coalesced one whatever K is.  Lane l of a group holds the classes l, l + G, l + 2G, ... and walks
// them from the `rot * row`-th on, wrapping round: the host picks rot (0 to 3) so that the lanes of a wave meet in
// different LDS banks (rows K floats apart would otherwise share banks whenever K / G is even).  The sum of a row
// is therefore taken in an order that depends on K and on the row number, and on nothing else.
template <int KMAX, int LOG2G, int NT>
__global__ __launch_bounds__(kBlock) void softmax_row_lds_kernel(uint32_t K, uint32_t R, uint32_t rot,
                                                                 FastDiv div_kj, int vec,
                                                                 const float *__restrict__ x,
                                                                 float *__restrict__ y, RowNll nl) {
  extern __shared__ __align__(16) float tile[];  // (kBlock >> LOG2G) * K floats, at most 32 KiB
  f32x4 *tile4 = reinterpret_cast<f32x4 *>(tile);
  constexpr uint32_t G = 1u << LOG2G;
  constexpr uint32_t rows_per_block = uint32_t(kBlock) >> LOG2G;
  const uint32_t KJ = div_kj.d;                    // ceil(K / G): values a lane may hold
  const uint32_t local = threadIdx.x >> LOG2G;     // row of the tile
  const uint32_t l = threadIdx.x & (G - 1u);       // lane of the row's group
  uint32_t q0, first;
  div_kj.divmod(local * rot, q0, first);           // where this row's walk starts
  for (uint64_t r0 = uint64_t(blockIdx.x) * rows_per_block; r0 < R; r0 += uint64_t(gridDim.x) * rows_per_block) {
    const uint32_t rows = (R - r0 < uint64_t(rows_per_block)) ? uint32_t(R - r0) : rows_per_block;
    const uint32_t n = rows * K;
    const float *xt = x + r0 * K;
    float *yt = y + r0 * K;
    // (the tile starts a multiple of 32 rows, hence a whole number of 16-byte groups, into the array)
    const uint32_t n4 = vec ? n / 4u : 0u;
    // the row's label and upstream gradient are requested together with the tile
    const uint64_t r = r0 + local;
    const bool mine = local < rows;  // the same for all lanes of a row's group
    const uint32_t label = (mine && nl.on()) ? nl.label(r) : 0u;
    const float dyr = (mine && nl.on() && nl.dx != nullptr) ? nl.dy[r] : 0.0f;
    if (n4 != 0u) {
      // the tile is at most 2048 groups, eight per thread: all requested before the first is written to LDS (a
      // slot past the tile's end reads its last group again and is dropped)
      f32x4 in[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t g = threadIdx.x + uint32_t(i) * kBlock;
        in[i] = load_stream<0>(reinterpret_cast<const f32x4 *>(xt) + (g < n4 ? g : n4 - 1u));
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t g = threadIdx.x + uint32_t(i) * kBlock;
        if (g < n4) tile4[g] = in[i];
      }
    }
    for (uint32_t e = n4 * 4u + threadIdx.x; e < n; e += kBlock) tile[e] = xt[e];
    __syncthreads();
    float *row = tile + local * K + l;  // this lane's classes are row[0], row[G], row[2G], ...
    float v[KMAX];
    if (mine) {  // whole lane groups take this branch or skip it, so the exchanges below stay inside active lanes
      float m = kNegInf;
      uint32_t at = first;
#pragma unroll
      for (int j = 0; j < KMAX; ++j) {
        if (uint32_t(j) < KJ) {
          v[j] = (G == 1u || l + (at << LOG2G) < K) ? row[at << LOG2G] : kNegInf;
          m = fmaxf(m, v[j]);
          at = (at + 1u == KJ) ? 0u : at + 1u;
        }
      }
      if (G > 1u) m = group_max(m, int(G));
      float sum = 0.0f;
#pragma unroll
      for (int j = 0; j < KMAX; ++j) {
        if (uint32_t(j) < KJ) {
          v[j] = exp_nonpos(v[j] - m);  // a slot past the row's end holds -inf and adds 0
          sum += v[j];
        }
      }
      if (G > 1u) sum = group_sum(sum, int(G));
      const float rsum = 1.0f / sum;  // one correctly rounded reciprocal per row
      at = first;
#pragma unroll
      for (int j = 0; j < KMAX; ++j) {
        if (uint32_t(j) < KJ) {
          v[j] = v[j] * rsum;
          if (G == 1u || l + (at << LOG2G) < K) row[at << LOG2G] = v[j];
          at = (at + 1u == KJ) ? 0u : at + 1u;
        }
      }
    }
    if (G > 1u) __syncthreads();  // the label's probability may have been written by another wave's lane
    if (mine && l == 0u && nl.on()) {
      const float *whole = tile + local * K;
      nl.emit_nll(r, K, label, label < K ? label : 0u, label < K ? whole[label] : 0.0f);
    }
    if (G == 1u) __syncthreads();
    for (uint32_t g = threadIdx.x; g < n4; g += kBlock) store_stream<NT>(reinterpret_cast<f32x4 *>(yt) + g, tile4[g]);
    for (uint32_t e = n4 * 4u + threadIdx.x; e < n; e += kBlock) yt[e] = tile[e];
    __syncthreads();  // the tile is overwritten below, or by the next pass
    if (nl.on() && nl.dx != nullptr) {
      // the gradient takes the same way out: each lane turns its classes into dy * (p - onehot) in place
      if (mine) {
        uint32_t at = first;
#pragma unroll
        for (int j = 0; j < KMAX; ++j) {
          if (uint32_t(j) < KJ) {
            const uint32_t k = l + (at << LOG2G);
            if (G == 1u || k < K) row[at << LOG2G] = RowNll::grad(dyr, label, k, v[j]);
            at = (at + 1u == KJ) ? 0u : at + 1u;
          }
        }
      }
      __syncthreads();
      float *dt = nl.dx + r0 * K;
      const uint32_t ad = vec ? uint32_t((reinterpret_cast<uintptr_t>(dt) >> 4) & 7u) : 0u;
      for (uint32_t slot = threadIdx.x; slot < n4 + ad; slot += kBlock) {
        if (slot >= ad) store_stream<NT>(reinterpret_cast<f32x4 *>(dt) + (slot - ad), tile4[slot - ad]);
      }
      for (uint32_t e = n4 * 4u + threadIdx.x; e < n; e += kBlock) dt[e] = tile[e];
      __syncthreads();
    }
  }
}

// The rotation (0 to 3 places per row) that spreads the first LDS access of a wave's 32-lane halves over most banks.
uint32_t pick_row_rotation(uint32_t K, uint32_t log2g) {
  const uint32_t G = 1u << log2g, KJ = (K + G - 1) / G;
  uint32_t best = 0, best_worst = ~0u;
  for (uint32_t rot = 0; rot < 4; ++rot) {
    uint32_t hits[32] = {0};
    uint32_t worst = 0;
    for (uint32_t t = 0; t < 32; ++t) {  // 32 lanes are served per cycle
      const uint32_t local = t >> log2g, l = t & (G - 1u);
      const uint32_t at = (local * rot) % KJ;
      uint32_t k = l + G * at;
      if (k >= K) k = l;  // such a lane sits the access out; count it where its next one goes
      const uint32_t bank = (local * K + k) % 32u;
      if (++hits[bank] > worst) worst = hits[bank];
    }
    if (worst < best_worst) {
      best_worst = worst;
      best = rot;
    }
  }
  return best;
}

// Up to 64 * VPL columns (from 225 on, see the dispatch): one wave per row, VPL values per lane.  VEC: rows are whole 16-byte groups (K a multiple
// of 4) and a lane owns groups of four consecutive classes; otherwise lane l owns k = l, l+64, ...
template <int VPL, bool VEC, int NT>
__global__ __launch_bounds__(kBlock) void softmax_row_wave_kernel(uint32_t K, uint32_t R,
                                                                  const float *__restrict__ x,
                                                                  float *__restrict__ y, RowNll nl) {
  constexpr int W = VEC ? 4 : 1;
  constexpr int NG = VPL / W;  // groups per lane
  static_assert((NG & (NG - 1)) == 0, "the wrapped lane assignment needs a power-of-two number of groups per lane");
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t wave = (blockIdx.x * kBlock + threadIdx.x) / kWave;
  const uint32_t n_waves = gridDim.x * (kBlock / kWave);
  for (uint64_t r = wave; r < R; r += n_waves) {
    const float *xr = x + size_t(r) * K;
    float *yr = y + size_t(r) * K;
    // VEC: step i of the wave covers one aligned run of 16-byte groups of the ARRAY, not of the row: the groups are
    // taken `a` places earlier, a = the row's distance from the 128-byte line before it (in groups, for an array
    // that starts on a line), and the first a lanes wrap round to the row's tail.  A row of 1000 floats starts 32
    // bytes into a line three times out of four, and half-written 64-byte pieces cost a tenth of the bandwidth
    // ([65536, 1000]: 5.5 TB/s, against 6.1 for 992 or 1024 columns).  The shift depends on the row number
    // only, so results do not depend on where the arrays lie.
    const uint32_t a = VEC ? (uint32_t(r) * (K / 4u)) & 7u : 0u;
    auto kof = [&](int i) -> uint32_t {
      const uint32_t slot = lane + uint32_t(i) * kWave;
      return VEC ? ((slot + uint32_t(NG) * kWave - a) & (uint32_t(NG) * kWave - 1u)) * 4u : slot;
    };
    // the row's label and upstream gradient are requested together with the row, not after the reductions
    const uint32_t label = nl.on() ? nl.label(r) : 0u;
    const float dyr = (nl.on() && nl.dx != nullptr) ? nl.dy[r] : 0.0f;
    float v[VPL];
    float m = kNegInf;
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const uint32_t k = kof(i);
      if (VEC) {
        const f32x4 t = (k < K) ? load_stream<NT>(reinterpret_cast<const f32x4 *>(xr + k))
                                : f32x4{kNegInf, kNegInf, kNegInf, kNegInf};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v[i * W + j] = t[j];
          m = fmaxf(m, t[j]);
        }
      } else {
        v[i] = (k < K) ? xr[k] : kNegInf;
        m = fmaxf(m, v[i]);
      }
    }
    m = wave_max(m);
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const uint32_t k = kof(i / W) + uint32_t(i % W);
      v[i] = (k < K) ? exp_nonpos(v[i] - m) : 0.0f;
      s += v[i];
    }
    s = wave_sum(s);
    const float rs = 1.0f / s;  // one correctly rounded reciprocal per row
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const uint32_t k = kof(i);
      if (k < K) {
#pragma unroll
        for (int j = 0; j < W; ++j) {
          v[i * W + j] = v[i * W + j] * rs;
          if (nl.on()) nl.emit_nll(r, K, label, k + uint32_t(j), v[i * W + j]);
        }
        if (VEC) {
          store_stream<NT>(reinterpret_cast<f32x4 *>(yr + k), f32x4{v[i * W], v[i * W + 1], v[i * W + 2], v[i * W + 3]});
          if (nl.on() && nl.dx != nullptr) {
            store_stream<NT>(reinterpret_cast<f32x4 *>(nl.dx + size_t(r) * K + k),
                             f32x4{RowNll::grad(dyr, label, k, v[i * W]), RowNll::grad(dyr, label, k + 1u, v[i * W + 1]),
                                   RowNll::grad(dyr, label, k + 2u, v[i * W + 2]),
                                   RowNll::grad(dyr, label, k + 3u, v[i * W + 3])});
          }
        } else {
          yr[k] = v[i];
          if (nl.on() && nl.dx != nullptr) nl.dx[size_t(r) * K + k] = RowNll::grad(dyr, label, k, v[i]);
        }
      }
    }
  }
}

// Merge two (max, sum-of-exp) pairs.  A side that has seen nothing carries
// (-inf, 0) and must not produce exp(-inf - -inf).
__device__ inline void online_merge(float &m, float &s, float m2, float s2) {
  const float mm = fmaxf(m, m2);
  const float a = (m == mm) ? s : s * exp_nonpos(m - mm);
  const float b = (m2 == mm) ? s2 : s2 * exp_nonpos(m2 - mm);
  s = ((s == 0.0f) ? 0.0f : a) + ((s2 == 0.0f) ? 0.0f : b);
  m = mm;
}

// 2048 < K <= THREADS * VPT: one workgroup per row, the row in registers (VPT values per thread), so x is read once.
// VEC as in the wave kernel.  THREADS is 256, or 1024 for rows of 16385 to 32768 classes (32 values per thread: the
// four waves that each SIMD then holds have 128 registers each, too few for 64 values without spilling).
template <int VPT, bool VEC, int NT, int THREADS = kBlock>
__global__ __launch_bounds__(THREADS) void softmax_row_blockreg_kernel(uint32_t K, uint32_t R,
                                                                      const float *__restrict__ x,
                                                                      float *__restrict__ y, RowNll nl) {
  constexpr int W = VEC ? 4 : 1;
  constexpr int NG = VPT / W;
  static_assert((NG & (NG - 1)) == 0, "the wrapped lane assignment needs a power-of-two number of groups per thread");
  __shared__ float lds[THREADS / kWave];
  for (uint64_t r = blockIdx.x; r < R; r += gridDim.x) {
    const float *xr = x + size_t(r) * K;
    float *yr = y + size_t(r) * K;
    // VEC: step i of the workgroup covers one aligned run of 16-byte groups of the ARRAY, not of the row: the groups are
    // taken `a` places earlier, a = the row's distance from the 128-byte line before it (in groups, for an array
    // that starts on a line), and the first a lanes wrap round to the row's tail.  A row of 1000 floats starts 32
    // bytes into a line three times out of four, and half-written 64-byte pieces cost a tenth of the bandwidth
    // ([65536, 1000]: 5.5 TB/s, against 6.1 for 992 or 1024 columns).  The shift depends on the row number
    // only, so results do not depend on where the arrays lie.
    const uint32_t a = VEC ? (uint32_t(r) * (K / 4u)) & 7u : 0u;
    auto kof = [&](int i) -> uint32_t {
      const uint32_t slot = threadIdx.x + uint32_t(i) * uint32_t(THREADS);
      return VEC ? ((slot + uint32_t(NG) * uint32_t(THREADS) - a) & (uint32_t(NG) * uint32_t(THREADS) - 1u)) * 4u : slot;
    };
    // the row's label and upstream gradient are requested together with the row, not after the reductions
    const uint32_t label = nl.on() ? nl.label(r) : 0u;
    const float dyr = (nl.on() && nl.dx != nullptr) ? nl.dy[r] : 0.0f;
    float v[VPT];
    float m = kNegInf;
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const uint32_t k = kof(i);
      if (VEC) {
        const f32x4 t = (k < K) ? load_stream<NT>(reinterpret_cast<const f32x4 *>(xr + k))
                                : f32x4{kNegInf, kNegInf, kNegInf, kNegInf};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v[i * W + j] = t[j];
          m = fmaxf(m, t[j]);
        }
      } else {
        v[i] = (k < K) ? xr[k] : kNegInf;
        m = fmaxf(m, v[i]);
      }
    }
    m = block_max<THREADS / kWave>(m, lds);
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const uint32_t k = kof(i / W) + uint32_t(i % W);
      v[i] = (k < K) ? exp_nonpos(v[i] - m) : 0.0f;
      s += v[i];
    }
    s = block_sum<float, THREADS / kWave>(s, lds);
    const float rs = 1.0f / s;  // one correctly rounded reciprocal per row
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const uint32_t k = kof(i);
      if (k < K) {
#pragma unroll
        for (int j = 0; j < W; ++j) {
          v[i * W + j] = v[i * W + j] * rs;
          if (nl.on()) nl.emit_nll(r, K, label, k + uint32_t(j), v[i * W + j]);
        }
        if (VEC) {
          store_stream<NT>(reinterpret_cast<f32x4 *>(yr + k), f32x4{v[i * W], v[i * W + 1], v[i * W + 2], v[i * W + 3]});
          if (nl.on() && nl.dx != nullptr) {
            store_stream<NT>(reinterpret_cast<f32x4 *>(nl.dx + size_t(r) * K + k),
                             f32x4{RowNll::grad(dyr, label, k, v[i * W]), RowNll::grad(dyr, label, k + 1u, v[i * W + 1]),
                                   RowNll::grad(dyr, label, k + 2u, v[i * W + 2]),
                                   RowNll::grad(dyr, label, k + 3u, v[i * W + 3])});
          }
        } else {
          yr[k] = v[i];
          if (nl.on() && nl.dx != nullptr) nl.dx[size_t(r) * K + k] = RowNll::grad(dyr, label, k, v[i]);
        }
      }
    }
  }
}

// Rows of up to 64 * THREADS classes in whole 16-byte groups, read once: one workgroup per row, the row's first half
// (the first 8 * THREADS slots) in LDS and its second half in registers, 32 values per thread each.  512 threads
// hold 32768 classes in 64 KB of LDS, so two workgroups fit a CU and one loads while the other reduces or stores
// (the register-only kernel above needs 1024 threads for such rows, one workgroup per CU, whose CU idles between its
// phases); 1024 threads hold 65536 classes in 128 KB of the CU's 160 KB, where the streaming kernel below keeps
// 16384 values and reads the rest a second time.  A thread's 16 slots are taken in two batches of eight 16-byte
// loads; the held half goes to LDS as it arrives, is read back for the sum of exponentials and once more for the
// normalised values.  Slots are dealt as in the register kernel (a step of the workgroup covers an aligned run of
// the array).  The row's sum is the workgroup sum of the threads' sums, each added in slot order, LDS half first.
template <int THREADS, int NT>
__global__ __launch_bounds__(THREADS) void softmax_row_reglds_kernel(uint32_t K, uint32_t R,
                                                                    const float *__restrict__ x,
                                                                    float *__restrict__ y, RowNll nl) {
  constexpr int NGH = 8;                           // groups per thread in each half
  constexpr uint32_t kSlots = 2u * NGH * THREADS;  // a power of two
  extern __shared__ __align__(16) float held_row[];  // NGH * THREADS groups of 16 bytes
  f32x4 *held = reinterpret_cast<f32x4 *>(held_row);
  __shared__ float lds[THREADS / kWave];
  for (uint64_t r = blockIdx.x; r < R; r += gridDim.x) {
    const float *xr = x + size_t(r) * K;
    float *yr = y + size_t(r) * K;
    float *dxr = (nl.on() && nl.dx != nullptr) ? nl.dx + size_t(r) * K : nullptr;
    const uint32_t a = (uint32_t(r) * (K / 4u)) & 7u;  // the row's distance in groups from a 128-byte line of the array
    auto kof = [&](int i) -> uint32_t {  // first class of slot i of this thread
      const uint32_t slot = threadIdx.x + uint32_t(i) * uint32_t(THREADS);
      return ((slot + kSlots - a) & (kSlots - 1u)) * 4u;
    };
    const uint32_t label = nl.on() ? nl.label(r) : 0u;
    const float dyr = dxr != nullptr ? nl.dy[r] : 0.0f;
    const f32x4 ninf = f32x4{kNegInf, kNegInf, kNegInf, kNegInf};
    float m = kNegInf;
    // first half: to LDS
    {
      f32x4 t[NGH];
#pragma unroll
      for (int i = 0; i < NGH; ++i) {
        const uint32_t k = kof(i);
        t[i] = (k < K) ? load_stream<NT>(reinterpret_cast<const f32x4 *>(xr + k)) : ninf;
      }
#pragma unroll
      for (int i = 0; i < NGH; ++i) {
        held[uint32_t(i) * THREADS + threadIdx.x] = t[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) m = fmaxf(m, t[i][j]);
      }
    }
    // second half: stays in registers
    f32x4 v[NGH];
#pragma unroll
    for (int i = 0; i < NGH; ++i) {
      const uint32_t k = kof(NGH + i);
      v[i] = (k < K) ? load_stream<NT>(reinterpret_cast<const f32x4 *>(xr + k)) : ninf;
    }
#pragma unroll
    for (int i = 0; i < NGH; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) m = fmaxf(m, v[i][j]);
    }
    m = block_max<THREADS / kWave>(m, lds);
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < NGH; ++i) {  // (a slot past the row's end holds -inf and adds exp(-inf - m) = 0, NaN only if m is)
      const f32x4 t = held[uint32_t(i) * THREADS + threadIdx.x];
      const bool in = kof(i) < K;
#pragma unroll
      for (int j = 0; j < 4; ++j) s += in ? exp_nonpos(t[j] - m) : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < NGH; ++i) {
      const bool in = kof(NGH + i) < K;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[i][j] = in ? exp_nonpos(v[i][j] - m) : 0.0f;
        s += v[i][j];
      }
    }
    s = block_sum<float, THREADS / kWave>(s, lds);
    const float rs = 1.0f / s;  // one correctly rounded reciprocal per row
    auto emit = [&](uint32_t k, f32x4 pr) {
      if (nl.on()) {
#pragma unroll
        for (int j = 0; j < 4; ++j) nl.emit_nll(r, K, label, k + uint32_t(j), pr[j]);
      }
      store_stream<NT>(reinterpret_cast<f32x4 *>(yr + k), pr);
      if (dxr != nullptr) {
        store_stream<NT>(reinterpret_cast<f32x4 *>(dxr + k),
                         f32x4{RowNll::grad(dyr, label, k, pr[0]), RowNll::grad(dyr, label, k + 1u, pr[1]),
                               RowNll::grad(dyr, label, k + 2u, pr[2]), RowNll::grad(dyr, label, k + 3u, pr[3])});
      }
    };
#pragma unroll
    for (int i = 0; i < NGH; ++i) {
      const uint32_t k = kof(NGH + i);
      if (k < K) emit(k, v[i] * rs);
    }
#pragma unroll
    for (int i = 0; i < NGH; ++i) {
      const uint32_t k = kof(i);
      if (k < K) {
        const f32x4 t = held[uint32_t(i) * THREADS + threadIdx.x];
        emit(k, vexp4(t - m) * rs);
      }
    }
  }
}

// any K: workgroups of 512 threads, two to a CU, each walking rows.  A row is taken in batches of U groups of W
// values per thread (a slot past the row's end reads the last group again and counts as -inf) and folded into a
// running maximum and a running sum of exponentials about it; the next batch is requested before the current one
// is folded, so the row streams in without a pause.  The first 16384 values are kept in LDS (64 KB) on the way,
// the rest is read again by the normalising pass, which is pipelined the same way; the next row's first batch is
// requested before the held part is written.  (One workgroup of 1024 threads per CU holding 32768 values was no
// faster: [2047, 32772] 3.3 TB/s against 4.0, [1024, 65536] 4.6 against 4.5.  A CU that loads, reduces and stores
// one row at a time leaves the memory system idle between the phases; two workgroups overlap them.)
constexpr int kRowStreamThreads = 512;
constexpr int kRowStreamHeld = 32 * kRowStreamThreads;  // values of a row that stay in LDS
// MODE 0: 4-byte accesses.  MODE 1: 16-byte accesses, every row is a whole number of 16-byte groups.  MODE 2: 16-byte
// accesses to the aligned groups of the array from the start of the 128-byte line of y in which a row begins (x and
// y, and dx, start equally far from a 16-byte boundary; `mis` is y's distance in floats from a line): every step of
// a wave then covers whole lines of y, whatever the row length, and the values of a row's first and last groups
// that belong to its neighbours are read, count as -inf and are not written (such a group is stored value by
// value).  `unit` is 32 floats, a line, where x lies in its line as y does in its own, and otherwise 4, one group:
// no load then reaches further back than the 16-byte group in which x begins.  Rows whose ends cut 64-byte pieces in two otherwise cost a fifth of the bandwidth: the two halves of a
// piece are written by different store instructions.  The order of a row's sum depends on where in a line the row
// starts.
// (four waves per SIMD, i.e. at most 128 registers: two workgroups must fit a CU)
template <int MODE, int NT>
__global__ __launch_bounds__(kRowStreamThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void softmax_row_stream_kernel(uint32_t K, uint32_t R, uint32_t mis,
                                                                               uint32_t unit,
                                                                               const float *__restrict__ x,
                                                                               float *__restrict__ y, RowNll nl) {
  constexpr bool VEC = MODE != 0;
  constexpr int THREADS = kRowStreamThreads;
  constexpr int W = VEC ? 4 : 1;
  constexpr int U = VEC ? 4 : 8;
  constexpr int WAVES = THREADS / kWave;
  constexpr uint32_t kBatch = uint32_t(THREADS) * U;  // groups per batch
  constexpr uint32_t kHeldBatches = uint32_t(kRowStreamHeld) / (kBatch * W);
  static_assert(kHeldBatches * kBatch * W == uint32_t(kRowStreamHeld), "whole batches are held");
  __shared__ __align__(16) float held[kRowStreamHeld];
  __shared__ float lds_m[WAVES], lds_s[WAVES];
  // A row's geometry: the `shift` values before it in its line come first (MODE 2 only), `groups` groups reach to
  // the row's end; group g holds the row's values 4 g - shift ... 4 g - shift + 3.
  struct RowGeom {
    const float *xa;  // the row's first group
    uint32_t shift, groups, batches, held_batches;
  };
  auto geom = [&](uint64_t r) {
    RowGeom g;
    g.shift = MODE == 2 ? uint32_t((uint64_t(mis) + r * K) & (unit - 1u)) : 0u;
    g.xa = x + size_t(r) * K - g.shift;
    g.groups = MODE == 2 ? uint32_t((uint64_t(K) + g.shift + 3u) / 4u) : K / uint32_t(W);  // MODE 1: K % 4 == 0
    g.batches = uint32_t((uint64_t(g.groups) + kBatch - 1u) / kBatch);
    g.held_batches = g.batches < kHeldBatches ? g.batches : kHeldBatches;
    return g;
  };
  // The values of group g that are the row's: j_lo <= j < j_hi.  (None for a group past the row's end; in MODE 2
  // the first groups hold the `shift` values before the row, and the last group may end with values of the row
  // after.)
  struct InRow {
    uint32_t j_lo, j_hi;
    __device__ bool operator()(int j) const { return uint32_t(j) >= j_lo && uint32_t(j) < j_hi; }
    __device__ bool none() const { return j_lo >= j_hi; }
    __device__ bool all() const { return j_lo == 0u && j_hi == uint32_t(W); }
  };
  auto in_row = [&](const RowGeom &rg, uint64_t g) {
    InRow v;
    if (MODE != 2) {
      v.j_lo = 0u;
      v.j_hi = g < rg.groups ? uint32_t(W) : 0u;
    } else {
      const uint64_t first = g * 4u, end = uint64_t(K) + rg.shift;  // in values counted from the line's start
      v.j_lo = first >= rg.shift ? 0u : (rg.shift - first < 4u ? uint32_t(rg.shift - first) : 4u);
      v.j_hi = first >= end ? 0u : (end - first < 4u ? uint32_t(end - first) : 4u);
    }
    return v;
  };
  // every value of group g is the row's (MODE 2)
  auto inside = [&](const RowGeom &rg, uint64_t g) { return g * 4u >= rg.shift && g * 4u + 4u <= uint64_t(K) + rg.shift; };
  // 64-bit group numbers: a batch's first group plus the batch can pass 2^32.  A batch past the row's end is
  // requested like any other (it reads the row's last group) and counts for nothing.
  auto request = [&](const RowGeom &rg, uint32_t b, float (&t)[U][W], auto last_use) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint64_t g = uint64_t(b) * kBatch + uint32_t(u) * uint32_t(THREADS) + threadIdx.x;
      const uint32_t gc = g < rg.groups ? uint32_t(g) : rg.groups - 1u;
      if (VEC) {
        const f32x4 q = decltype(last_use)::value ? load_stream<NT>(reinterpret_cast<const f32x4 *>(rg.xa + size_t(gc) * 4u))
                                                  : load_stream<0>(reinterpret_cast<const f32x4 *>(rg.xa + size_t(gc) * 4u));
#pragma unroll
        for (int j = 0; j < W; ++j) t[u][j] = q[j];
      } else {
        t[u][0] = rg.xa[gc];
      }
    }
  };
  float ta[U][W], tb[U][W];
  RowGeom rg = geom(blockIdx.x < R ? blockIdx.x : 0u);
  if (blockIdx.x < R) request(rg, 0, ta, std::false_type{});
  for (uint64_t r = blockIdx.x; r < R; r += gridDim.x) {
    float *ya = y + size_t(r) * K - rg.shift;
    float *dxa = (nl.on() && nl.dx != nullptr) ? nl.dx + size_t(r) * K - rg.shift : nullptr;
    const uint32_t label = nl.on() ? nl.label(r) : 0u;
    const float dyr = (nl.on() && nl.dx != nullptr) ? nl.dy[r] : 0.0f;
    const uint32_t batches = rg.batches, held_batches = rg.held_batches;
    // the held batches: slot (b * U + u) * THREADS + threadIdx.x, written and read by the same thread
    auto keep = [&](uint32_t b, const float (&t)[U][W]) {
      if (b >= held_batches) return;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t slot = (b * uint32_t(U) + uint32_t(u)) * uint32_t(THREADS) + threadIdx.x;
        if (VEC) {
          reinterpret_cast<f32x4 *>(held)[slot] = f32x4{t[u][0], t[u][1], t[u][2], t[u][3]};
        } else {
          held[slot] = t[u][0];
        }
      }
    };
    auto recall = [&](uint32_t b, float (&t)[U][W]) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t slot = (b * uint32_t(U) + uint32_t(u)) * uint32_t(THREADS) + threadIdx.x;
        if (VEC) {
          const f32x4 q = reinterpret_cast<const f32x4 *>(held)[slot];
#pragma unroll
          for (int j = 0; j < W; ++j) t[u][j] = q[j];
        } else {
          t[u][0] = held[slot];
        }
      }
    };
    float m = kNegInf, s = 0.0f;
    auto fold = [&](uint32_t b, float (&t)[U][W]) {
      float bm = kNegInf;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint64_t g = uint64_t(b) * kBatch + uint32_t(u) * uint32_t(THREADS) + threadIdx.x;
        // MODE 2: a wave whose groups all lie inside the row (all but the waves at a row's two ends) masks nothing
        if (MODE == 2 && __all(inside(rg, g))) {
#pragma unroll
          for (int j = 0; j < W; ++j) bm = fmaxf(bm, t[u][j]);
        } else {
          const InRow mine = in_row(rg, g);
#pragma unroll
          for (int j = 0; j < W; ++j) {
            if (!mine(j)) t[u][j] = kNegInf;
            bm = fmaxf(bm, t[u][j]);
          }
        }
      }
      float bs = 0.0f;
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int j = 0; j < W; ++j) bs += exp_nonpos(t[u][j] - bm);
      }
      if (bm == kNegInf) {
        // a batch of -inf has seen nothing: its sum, exp(-inf - -inf) = NaN, is not a sum.  A NaN among them
        // (which the maximum ignores) still has to reach the row's sum.
        bool nan = false;
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
          for (int j = 0; j < W; ++j) nan |= t[u][j] != t[u][j];
        }
        bs = nan ? __builtin_nanf("") : 0.0f;
      }
      online_merge(m, s, bm, bs);
    };
    float rs = 0.0f;
    auto write = [&](uint32_t b, float (&t)[U][W]) {
#pragma unroll
      for (int u = 0; u < U; ++u) {  // all of the batch is known to be there before the first store is issued
#pragma unroll
        for (int j = 0; j < W; ++j) arrived(t[u][j]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint64_t g = uint64_t(b) * kBatch + uint32_t(u) * uint32_t(THREADS) + threadIdx.x;
        InRow mine;
        if (MODE == 2 && __all(inside(rg, g))) {
          mine.j_lo = 0u;
          mine.j_hi = uint32_t(W);
        } else {
          mine = in_row(rg, g);
        }
        if (!mine.none()) {
          // the row's value number of the group's first value; "negative" (wrapped) for the values of a first group
          // that belong to the row before, which `mine` leaves out
          const uint32_t k = uint32_t(g) * uint32_t(W) - rg.shift;
#pragma unroll
          for (int j = 0; j < W; ++j) {
            t[u][j] = exp_nonpos(t[u][j] - m) * rs;
            if (nl.on() && mine(j)) nl.emit_nll(r, K, label, k + uint32_t(j), t[u][j]);
          }
          if (VEC) {
            if (mine.all()) {
              store_stream<NT>(reinterpret_cast<f32x4 *>(ya + size_t(g) * 4u), f32x4{t[u][0], t[u][1], t[u][2], t[u][3]});
              if (dxa != nullptr) {  // the host checked that dx lies like y
                store_stream<NT>(reinterpret_cast<f32x4 *>(dxa + size_t(g) * 4u),
                                 f32x4{RowNll::grad(dyr, label, k, t[u][0]), RowNll::grad(dyr, label, k + 1u, t[u][1]),
                                       RowNll::grad(dyr, label, k + 2u, t[u][2]),
                                       RowNll::grad(dyr, label, k + 3u, t[u][3])});
              }
            } else {
#pragma unroll
              for (int j = 0; j < W; ++j) {
                if (mine(j)) {
                  ya[size_t(g) * 4u + uint32_t(j)] = t[u][j];
                  if (dxa != nullptr) dxa[size_t(g) * 4u + uint32_t(j)] = RowNll::grad(dyr, label, k + uint32_t(j), t[u][j]);
                }
              }
            }
          } else {
            ya[g] = t[u][0];
            if (dxa != nullptr) dxa[g] = RowNll::grad(dyr, label, k, t[u][0]);
          }
        }
      }
    };
    // ta holds the row's first batch: requested before the loop for the workgroup's first row, and by the
    // previous row before it began to store
#pragma unroll 1
    for (uint32_t b = 0; b < batches; b += 2) {
      request(rg, b + 1u, tb, std::false_type{});
      fold(b, ta);
      keep(b, ta);
      request(rg, b + 2u, ta, std::false_type{});
      fold(b + 1u, tb);
      keep(b + 1u, tb);
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      const float m2 = __shfl_xor(m, off, kWave);
      const float s2 = __shfl_xor(s, off, kWave);
      online_merge(m, s, m2, s2);
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
      lds_m[threadIdx.x / kWave] = m;
      lds_s[threadIdx.x / kWave] = s;
    }
    __syncthreads();
    m = lds_m[0];
    s = lds_s[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) online_merge(m, s, lds_m[w], lds_s[w]);
    __syncthreads();
    rs = 1.0f / s;
    if (held_batches < batches) {
      request(rg, held_batches, ta, std::true_type{});
#pragma unroll 1
      for (uint32_t b = held_batches; b < batches; b += 2) {
        request(rg, b + 1u, tb, std::true_type{});
        write(b, ta);
        request(rg, b + 2u, ta, std::true_type{});
        write(b + 1u, tb);
      }
    }
    // the next row starts to arrive while this one's held part is written
    const RowGeom next = geom(r + gridDim.x < R ? r + gridDim.x : r);
    if (r + gridDim.x < R) request(next, 0, ta, std::false_type{});
#pragma unroll 1
    for (uint32_t b = 0; b < held_batches; ++b) {
      recall(b, tb);
      write(b, tb);
    }
    rg = next;
  }
}

template <int THREADS, int NT>
void launch_softmax_row_reglds(uint32_t blocks, uint32_t K, uint32_t R, const float *x, float *y, const RowNll &nl,
                               hipStream_t s) {
  constexpr size_t lds_bytes = size_t(8) * THREADS * 16;
  // more than the 64 KB a kernel may take by default: raised once per device
  static std::atomic<bool> raised[64];
  int dev = 0;
  (void)hipGetDevice(&dev);
  if (dev >= 0 && dev < 64 && !raised[dev].load(std::memory_order_relaxed)) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&softmax_row_reglds_kernel<THREADS, NT>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
    raised[dev].store(true, std::memory_order_relaxed);
  }
  softmax_row_reglds_kernel<THREADS, NT><<<blocks, THREADS, lds_bytes, s>>>(K, R, x, y, nl);
}

void launch_softmax_rows(const char *symbol, uint32_t K, uint32_t R, const float *x, float *y,
                         CUstream_st *stream, RowNll nl = RowNll{nullptr, nullptr, false, nullptr, nullptr}) {
  (void)checked_len(K, R, 1, symbol);
  if (K == 0 || R == 0) return;
  hipStream_t s = as_stream(stream);
  // one row (or group of rows) per wave / workgroup and a grid that covers all of them: the loop in the kernels
  // only runs again when the row count exceeds the grid limit
  const uint32_t max_blocks = 1u << 24;
  constexpr uint32_t kWavesPerBlock = kBlock / kWave;
  // logits in, probabilities out: both streamed (streaming stores only for outputs that start on 64-byte boundaries)
  const int nt = policy_for_outputs(stream_policy(size_t(K) * R * sizeof(float), tuning().nontemporal), y, nl.dx);
  if (K <= 224 || (K <= 256 && K % 16u != 0)) {
    // 1, 2, 4 or 8 lanes per row, at most 32 values per lane; the tile of 256 / G rows is at most 32 KiB.
    // The kernel is built for 4, 8, 16, 20, 24, 28 or 32 values per lane: the registers of a lane's array are what
    // limits the waves per SIMD (K = 33 with room for 32 values per lane: 3.7 TB/s, for 20: 5.6).
    // (Rows of 240 and 256 columns go to the wave-per-row kernel below, whose lanes then all take whole 64-byte
    // pieces: 5.9 and 6.1 TB/s against 5.4 and 5.5 here; at 232 columns it runs at 4.9 against 5.4 here.)
    uint32_t log2g = 0;
    while ((32u << log2g) < K) ++log2g;
    const uint32_t G = 1u << log2g, KJ = (K + G - 1) / G;
    const uint32_t rows_per_block = uint32_t(kBlock) >> log2g;
    uint32_t blocks = (R + rows_per_block - 1) / rows_per_block;
    if (blocks > max_blocks) blocks = max_blocks;
    const size_t lds_bytes = size_t(rows_per_block) * K * sizeof(float);
    const FastDiv div_kj(KJ);
    const uint32_t rot = pick_row_rotation(K, log2g);
    const int vec = 1;  // 16-byte copies between the arrays and the tile, wherever the arrays lie (4-byte aligned accesses)
    with_stream_policy(nt & kNtStore, [&](auto policy) {
      constexpr int NT = decltype(policy)::value;
      auto launch = [&](auto kmax, auto lg) {
        softmax_row_lds_kernel<decltype(kmax)::value, decltype(lg)::value, NT>
            <<<blocks, kBlock, lds_bytes, s>>>(K, R, rot, div_kj, vec, x, y, nl);
      };
      auto with_kmax = [&](auto lg) {
        if (KJ <= 4) {
          launch(std::integral_constant<int, 4>{}, lg);
        } else if (KJ <= 8) {
          launch(std::integral_constant<int, 8>{}, lg);
        } else if (KJ <= 16) {
          launch(std::integral_constant<int, 16>{}, lg);
        } else {
          launch(std::integral_constant<int, 32>{}, lg);
        }
      };
      auto with_kmax_wide = [&](auto lg) {  // several lanes per row: 17 to 32 values per lane
        if (KJ <= 20) {
          launch(std::integral_constant<int, 20>{}, lg);
        } else if (KJ <= 24) {
          launch(std::integral_constant<int, 24>{}, lg);
        } else if (KJ <= 28) {
          launch(std::integral_constant<int, 28>{}, lg);
        } else {
          launch(std::integral_constant<int, 32>{}, lg);
        }
      };
      if (log2g == 0) {
        with_kmax(std::integral_constant<int, 0>{});
      } else if (log2g == 1) {
        with_kmax_wide(std::integral_constant<int, 1>{});
      } else if (log2g == 2) {
        with_kmax_wide(std::integral_constant<int, 2>{});
      } else {
        with_kmax_wide(std::integral_constant<int, 3>{});
      }
    });
  } else if (K <= 2048 && K > 512 && R <= 2u * uint32_t(device_cu_count()) && (K % 4u == 0)) {
    // few rows: a workgroup per row instead of a wave, so that every CU has work ([256, 1000], launch-bound:
    // softmax + NLL + backward 8.2 -> 7.4 us as three launches inside a graph, 4.3 -> 3.8 us as one)
    with_stream_policy(nt, [&](auto policy) {
      if (K <= 1024) {
        softmax_row_blockreg_kernel<4, true, decltype(policy)::value, kBlock><<<R, kBlock, 0, s>>>(K, R, x, y, nl);
      } else {
        softmax_row_blockreg_kernel<8, true, decltype(policy)::value, kBlock><<<R, kBlock, 0, s>>>(K, R, x, y, nl);
      }
    });
  } else if (K <= 2048) {
    uint32_t blocks = (R + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > max_blocks) blocks = max_blocks;
    const bool vec = (K % 4u == 0);  // rows of whole 16-byte groups, wherever the arrays lie
#define ANODE_ROW_WAVE(VPL)                                                              \
  do {                                                                                   \
    if (vec) {                                                                           \
      with_stream_policy(nt, [&](auto policy) {                                          \
        softmax_row_wave_kernel<VPL, true, decltype(policy)::value><<<blocks, kBlock, 0, s>>>(K, R, x, y, nl); \
      });                                                                                \
    } else {                                                                             \
      softmax_row_wave_kernel<VPL, false, 0><<<blocks, kBlock, 0, s>>>(K, R, x, y, nl);  \
    }                                                                                    \
  } while (0)
    if (K <= 256) {
      ANODE_ROW_WAVE(4);
    } else if (K <= 512) {
      ANODE_ROW_WAVE(8);
    } else if (K <= 1024) {
      ANODE_ROW_WAVE(16);
    } else {
      ANODE_ROW_WAVE(32);
    }
#undef ANODE_ROW_WAVE
  } else {
    const uint32_t blocks = R < max_blocks ? R : max_blocks;
    const bool vec = (K % 4u == 0);  // rows of whole 16-byte groups, wherever the arrays lie
#define ANODE_ROW_BLOCKREG(VPT)                                                          \
  do {                                                                                   \
    if (vec) {                                                                           \
      with_stream_policy(nt, [&](auto policy) {                                          \
        softmax_row_blockreg_kernel<VPT, true, decltype(policy)::value><<<blocks, kBlock, 0, s>>>(K, R, x, y, nl); \
      });                                                                                \
    } else {                                                                             \
      softmax_row_blockreg_kernel<VPT, false, 0><<<blocks, kBlock, 0, s>>>(K, R, x, y, nl); \
    }                                                                                    \
  } while (0)
    if (K <= 4096) {
      ANODE_ROW_BLOCKREG(16);
    } else if (K <= 8192) {
      ANODE_ROW_BLOCKREG(32);
    } else if (K <= (vec ? 9216u : 8192u)) {  // (with 4-byte accesses 64 values per thread take 210 registers: [8191, 8193] 3.7 TB/s)
      ANODE_ROW_BLOCKREG(64);
    } else if (K <= 16384) {
      // workgroups of 512 threads, 32 values each: two to a CU with four waves per SIMD, where 256 threads of 64
      // values leave two ([4096, 16384] 5.2 -> 5.6 TB/s, [5460, 12289] 4.3 -> 5.0; [8188, 8196] 5.8 against 5.6)
      if (vec) {
        with_stream_policy(nt, [&](auto policy) {
          softmax_row_blockreg_kernel<32, true, decltype(policy)::value, 512><<<blocks, 512, 0, s>>>(K, R, x, y, nl);
        });
      } else {
        softmax_row_blockreg_kernel<32, false, 0, 512><<<blocks, 512, 0, s>>>(K, R, x, y, nl);
      }
    } else if (vec && K <= 32768 && (tuning().row_reglds & 1)) {
      // workgroups of 512 threads, two to a CU: half of the row in LDS, half in registers ([2730, 24576] 4.8 -> 5.8
      // TB/s, [2048, 32768] 4.9 -> 5.5 against 1024 threads with the whole row in registers, one workgroup per CU)
      with_stream_policy(nt, [&](auto policy) { launch_softmax_row_reglds<512, decltype(policy)::value>(blocks, K, R, x, y, nl, s); });
    } else if (vec && K <= 65536 && (tuning().row_reglds & 2)) {
      // one workgroup of 1024 threads per CU: half of the row in 128 KB of LDS, half in registers; x is read once
      // ([1335, 50256] 4.2 -> 4.6 TB/s, [1024, 65536] 4.65 -> 5.05, [2047, 32772] 4.1 -> 4.6 against the streaming
      // kernel below; [1864, 36000] and [1677, 40000] 4.5 and 4.7 either way)
      const uint32_t cus = uint32_t(device_cu_count());
      with_stream_policy(nt, [&](auto policy) {
        launch_softmax_row_reglds<1024, decltype(policy)::value>(R < cus ? R : cus, K, R, x, y, nl, s);
      });
    } else if (!vec && K <= 32768) {
      // rows that are not whole 16-byte groups: workgroups of 1024 threads, 32 values each, 4-byte accesses
      softmax_row_blockreg_kernel<32, false, 0, 1024><<<blocks, 1024, 0, s>>>(K, R, x, y, nl);
    } else {
      // two workgroups per CU, which walk their rows
      const uint32_t cus = 2u * uint32_t(device_cu_count());
      const uint32_t walkers = R < cus ? R : cus;
      // Rows that do not start on 128-byte lines are read and written in the array's 16-byte groups, from the
      // start of y's line, where x and y (and dx) start equally far from a 16-byte boundary.
      const auto floats_past = [](const float *p, uint32_t unit) { return uint32_t((reinterpret_cast<uintptr_t>(p) >> 2) & (unit - 1u)); };
      const auto lies_like_y = [&](const float *p) { return floats_past(p, 4) == floats_past(y, 4); };
      const bool floats = (reinterpret_cast<uintptr_t>(x) & 3u) == 0 && (reinterpret_cast<uintptr_t>(y) & 3u) == 0;
      if (vec) {
        with_stream_policy(nt, [&](auto policy) {
          softmax_row_stream_kernel<1, decltype(policy)::value>
              <<<walkers, kRowStreamThreads, 0, s>>>(K, R, 0u, 1u, x, y, nl);
        });
      } else if (floats && lies_like_y(x) && (nl.dx == nullptr || lies_like_y(nl.dx))) {
        const uint32_t unit = floats_past(x, 32) == floats_past(y, 32) ? 32u : 4u;
        with_stream_policy(nt, [&](auto policy) {
          softmax_row_stream_kernel<2, decltype(policy)::value>
              <<<walkers, kRowStreamThreads, 0, s>>>(K, R, floats_past(y, unit), unit, x, y, nl);
        });
      } else {
        softmax_row_stream_kernel<0, 0><<<walkers, kRowStreamThreads, 0, s>>>(K, R, 0u, 1u, x, y, nl);
      }
    }
#undef ANODE_ROW_BLOCKREG
  }
  note_launch(symbol);
}

// softmax.cu:144-161  nll[i] = label < K ? -log(p[label + K*i]) : NaN
__global__ __launch_bounds__(kBlock) void softmax_cat_nll_kernel(uint32_t K, uint32_t R,
                                                                 const float *__restrict__ p,
                                                                 const uint32_t *__restrict__ cat,
                                                                 float *__restrict__ nll, bool ignore) {
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;  // 64-bit: index + stride can pass 2^32
  for (uint64_t i = uint64_t(blockIdx.x) * kBlock + threadIdx.x; i < R; i += stride) {
    const uint32_t k = cat[i];
    nll[i] = (k < K) ? -logf(p[size_t(k) + size_t(K) * i]) : (ignore ? 0.0f : __builtin_nanf(""));
  }
}

// softmax.cu:177-195  dx[k,i] (=|+=) dy[i] * (p[k,i] - float(label[i]==k)); as a
// channel-indexed map the "channel" is the row i and s is the class k.
// With ignore set, a row whose label is >= n_classes gets dy = 0 (the "ignore" variants); the reference's
// semantics leaves the gradient unmasked.
struct CatNllBwdMap {
  const float *dy;
  const uint32_t *cat;
  uint32_t n_classes;
  bool ignore;
  struct Param { float dy; uint32_t label; };
  __device__ Param load(uint32_t i) const {
    const uint32_t label = cat[i];
    return Param{(ignore && label >= n_classes) ? 0.0f : dy[i], label};
  }
  __device__ float value(const Param &p, float prob, float, uint32_t k) const {
    return p.dy * (prob - float(p.label == k));
  }
  __device__ float accum(const Param &p, float prob, float, uint32_t k, float old) const {
    return fmaf(p.dy, prob - float(p.label == k), old);
  }
};

// ---------------------------------------------------------------------------
// N-d (channel-axis) softmax: one thread per group of W consecutive pixels
// ---------------------------------------------------------------------------

template <typename V> struct PixVec;
template <> struct PixVec<float> {
  static constexpr int W = 1;
  typedef uint32_t U;
  static __device__ float splat(float v) { return v; }
};
template <> struct PixVec<f32x4> {
  static constexpr int W = 4;
  typedef u32x4 U;
  static __device__ f32x4 splat(float v) { return f32x4{v, v, v, v}; }
};

__device__ inline uint32_t lane_get_u(uint32_t v, int) { return v; }
__device__ inline uint32_t lane_get_u(u32x4 v, int k) { return v[k]; }

__device__ inline float vexp(float a) { return exp_nonpos(a); }
__device__ inline f32x4 vexp(f32x4 a) { return f32x4{exp_nonpos(a.x), exp_nonpos(a.y), exp_nonpos(a.z), exp_nonpos(a.w)}; }
__device__ inline float vrcp(float a) { return 1.0f / a; }
__device__ inline f32x4 vrcp(f32x4 a) { return f32x4{1.0f / a.x, 1.0f / a.y, 1.0f / a.z, 1.0f / a.w}; }

// Pixel-group geometry shared by the N-d kernels: group g covers pixels
// [W*pg, W*pg + W) of sample n, with g = pg + groups_per_sample * n.  Where W does not divide P, the last group of a
// plane is moved back to end with the plane: it covers the plane's last W pixels, some of which the group before it
// covers too (both compute and store the same values for those; the arrays must not alias, and P >= W).
struct PixelGrid {
  uint32_t P, C, N;
  uint32_t total_groups;
  uint32_t ignore;  // 1: an out-of-range label gives nll = 0 and no gradient, instead of NaN and dy * p
  uint32_t xcd;     // 1: pixel groups are dealt to the XCDs in contiguous ranges (xcd_contiguous)
  FastDiv div_gps;  // groups per sample
};

__device__ inline void pixel_decode(const PixelGrid &pg, uint32_t g, int W, uint32_t &p, uint32_t &n) {
  uint32_t q, r;
  pg.div_gps.divmod(g, q, r);
  n = q;
  p = r * uint32_t(W);
  if (pg.P - p < uint32_t(W)) p = pg.P - uint32_t(W);  // (p < P)
}


// the value held by the lane whose number differs in the bits of `off`
__device__ inline float lane_swap(float v, int off) { return __shfl_xor(v, off, kWave); }
__device__ inline f32x4 lane_swap(f32x4 v, int off) {
  return f32x4{__shfl_xor(v.x, off, kWave), __shfl_xor(v.y, off, kWave), __shfl_xor(v.z, off, kWave),
               __shfl_xor(v.w, off, kWave)};
}

// C <= CMAX: the pixel's classes stay in registers, x is read once.  SPLIT lanes (1, 2 or 8) share a group of W
// pixels: lane h of the group holds classes h, h + SPLIT, ... and the group's maxima and sums meet through lane
// exchanges.  Two lanes per group halve a thread's state (ten 16-byte loads in flight instead of nineteen at
// C = 19) and measured 112 us against 120 us at [512K, 19, 8]; four or eight lanes are slower there (118, 122 us:
// a load instruction then covers several short runs), but they are what keeps 33 to 256 classes in registers.
// A lane adds its exponentials in class order, the group's sums are added last; the normalisation multiplies by one correctly rounded reciprocal per pixel.  With NLL the label
// gather is fused: nll = -log(the stored probability of the label), NaN when the label is out of range, exactly
// what the separate gather returns.
// With BWD the gradient of the summed loss for a dy known up front is written in the same pass:
// dx = dy * (p - onehot), the arithmetic (and, with pg.ignore, the masking) of softmax_nd_cat_nll_bwd_kernel.
// (With the backward pass the 20-class form takes 129 registers, one more than four waves per SIMD leave.  Held to
// 128 it measures the same, 182 us at [512K, 19, 8] in a process that holds nothing else, 204 against 201 among
// the other arrays of the benchmark: the kernel waits for memory, not for a free wave slot.)
template <int CMAX, typename V, bool NLL, int NT, int SPLIT, bool BWD = false>
__global__ __launch_bounds__(kBlock) void softmax_nd_reg_kernel(PixelGrid pg, const float *__restrict__ x,
                                                                float *__restrict__ y,
                                                                const uint32_t *__restrict__ cat,
                                                                float *__restrict__ nll,
                                                                const float *__restrict__ dy = nullptr,
                                                                float *__restrict__ dx = nullptr) {
  static_assert(!BWD || NLL, "the backward pass needs the labels");
  constexpr int W = PixVec<V>::W;
  constexpr int H = (CMAX + SPLIT - 1) / SPLIT;  // classes a lane holds
  typedef typename PixVec<V>::U U;
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;  // 64-bit: index + stride can pass 2^32
  const uint64_t total = uint64_t(pg.total_groups) * SPLIT;
  for (uint64_t t = uint64_t(pg.xcd ? xcd_contiguous(blockIdx.x, gridDim.x) : blockIdx.x) * kBlock + threadIdx.x; t < total; t += stride) {
    // the lanes of a pair are neighbours (t even, t + 1), so they always run, and leave the loop, together
    const uint32_t g = uint32_t(t / SPLIT), h = uint32_t(t % SPLIT);
    uint32_t p, n;
    pixel_decode(pg, uint32_t(g), W, p, n);  // g < total_groups, which fits 32 bits
    const size_t base = size_t(p) + size_t(pg.P) * pg.C * n;
    const size_t pix = size_t(p) + size_t(pg.P) * n;
    // the labels and the upstream gradient are requested first, so that they are there when the classes are
    U lab;
    if (NLL) lab = load_stream<0>(reinterpret_cast<const U *>(cat + pix));
    V d;
    if (BWD) d = load_stream<0>(reinterpret_cast<const V *>(dy + pix));
    if (NLL) issue_order_fence();
    // Every slot is loaded, a slot past the last class from the last class's plane again (and set to -inf below):
    // with a branch round each load the compiler waits for the previous load before it issues the next one.
    V v[H];
#pragma unroll
    for (int i = 0; i < H; ++i) {
      const uint32_t k = uint32_t(i) * SPLIT + h;
      const uint32_t kk = k < pg.C ? k : pg.C - 1u;
      v[i] = load_stream<NT>(reinterpret_cast<const V *>(x + base + size_t(pg.P) * kk));
    }
    if (NLL) arrived(lab);
    if (BWD) {
      arrived(d);
      if (pg.ignore) {
#pragma unroll
        for (int w = 0; w < W; ++w) {
          if (lane_get_u(lab, w) >= pg.C) lane_set<V>(d, w, 0.0f);
        }
      }
    }
    V m = PixVec<V>::splat(kNegInf);
#pragma unroll
    for (int i = 0; i < H; ++i) {
      if (uint32_t(i) * SPLIT + h >= pg.C) v[i] = PixVec<V>::splat(kNegInf);
      m = vmax(m, v[i]);
    }
#pragma unroll
    for (int off = 1; off < SPLIT; off <<= 1) m = vmax(m, lane_swap(m, off));
    V s = PixVec<V>::splat(0.0f);
#pragma unroll
    for (int i = 0; i < H; ++i) {
      // a slot past the last class holds -inf and adds exp(-inf - m) = 0 (NaN only where m is -inf or NaN, and
      // then the pixel's own classes give NaN as well)
      v[i] = vexp(v[i] - m);
      s += v[i];
    }
#pragma unroll
    for (int off = 1; off < SPLIT; off <<= 1) s += lane_swap(s, off);  // a + b == b + a: every lane holds the same sum
    const V inv = vrcp(s);
#pragma unroll
    for (int i = 0; i < H; ++i) {
      const uint32_t k = uint32_t(i) * SPLIT + h;
      if (k < pg.C) {
        const V pr = v[i] * inv;
        store_stream<NT>(reinterpret_cast<V *>(y + base + size_t(pg.P) * k), pr);
        if (BWD) {
          V gr;
#pragma unroll
          for (int w = 0; w < W; ++w) {
            lane_set<V>(gr, w, lane_get<V>(d, w) * (lane_get<V>(pr, w) - float(lane_get_u(lab, w) == k)));
          }
          store_stream<NT>(reinterpret_cast<V *>(dx + base + size_t(pg.P) * k), gr);
        }
      }
    }
    if (NLL) {
      // The label's exponential is picked out of the registers of the lane that holds it (a compare and a select
      // per held class and pixel) and handed to lane 0 of the pair, which multiplies it by the reciprocal as the
      // stored probability was.  (Reading the label's logit again instead, one 4-byte gather per pixel of a line
      // the wave had just requested, took 169 us against 109 us without NLL at [512K, 19, 8].)
      V pick = PixVec<V>::splat(0.0f);
#pragma unroll
      for (int i = 0; i < H; ++i) {
#pragma unroll
        for (int w = 0; w < W; ++w) {
          const uint32_t lb = lane_get_u(lab, w);
          if (lb / uint32_t(SPLIT) == uint32_t(i) && lb % uint32_t(SPLIT) == h) lane_set<V>(pick, w, lane_get<V>(v[i], w));
        }
      }
      // one lane of the group holds the label's exponential, the others hold 0: the sum hands it to all of them
#pragma unroll
      for (int off = 1; off < SPLIT; off <<= 1) pick += lane_swap(pick, off);
      if (h == 0) {
        V out;
#pragma unroll
        for (int w = 0; w < W; ++w) {
          const float pr = lane_get<V>(pick, w) * lane_get<V>(inv, w);
          lane_set<V>(out, w, lane_get_u(lab, w) < pg.C ? -logf(pr) : (pg.ignore ? 0.0f : __builtin_nanf("")));
        }
        store_stream<0>(reinterpret_cast<V *>(nll + pix), out);
      }
    }
  }
}

// The two-lanes-per-pixel-group form of the kernel above (16-byte accesses, up to 32 classes) with wave-uniform
// plane addresses.  A wave's 32 pixel groups lie a few hundred bytes apart (further only where the wave crosses
// from one sample into the next), so every access is "the plane's address for the wave's first group", a scalar
// pair computed on the scalar unit, plus one 32-bit byte offset per lane that is the same for all planes of an
// array.  The kernel above keeps a 64-bit address per plane and lane in vector registers instead: 129 registers
// with the backward pass (three waves per SIMD), 104 to 110 without; this form takes 68 (seven waves per SIMD) and
// no address arithmetic on the vector unit.  [512K, 19, 8] with NLL and backward: 194 -> 175 us among the other
// arrays of a training step, 181 -> 174 us alone.  One pixel group per lane pair and no loop: the grid covers the
// array.  With the backward pass the probabilities are stored first, plane after plane, then the gradient
// (measured against storing both for each plane in turn: 174 against 179 us).
// The arithmetic and the order of every sum are those of the kernel above: the two give the same bits.
// OFF is the type of the lane offset: uint32_t wherever a wave's byte offsets fit 32 bits (the host checks
// nd_pair_offsets_fit()), uint64_t otherwise (samples of a gigabyte and more), which costs the scalar base.
template <typename OFF>
__device__ inline f32x4 load_lane_off(const float *wave_base, OFF off, std::integral_constant<int, 0>) {
  return load_stream<0>(reinterpret_cast<const f32x4 *>(reinterpret_cast<const char *>(wave_base) + off));
}
template <typename OFF>
__device__ inline f32x4 load_lane_off(const float *wave_base, OFF off, std::integral_constant<int, kNtLoad>) {
  return __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(reinterpret_cast<const char *>(wave_base) + off));
}
template <int NT, typename OFF>
__device__ inline void store_lane_off(float *wave_base, OFF off, f32x4 v) {
  if constexpr ((NT & kNtStore) != 0 && sizeof(OFF) == 4) {
    // store_stream()'s instruction in its scalar-base form (see there for the policy bits and the s_nop)
    asm volatile("global_store_dwordx4 %0, %1, %2 sc1 nt\n\ts_nop 1" : : "v"(off), "v"(v), "s"(wave_base) : "memory");
  } else {
    store_stream<NT>(reinterpret_cast<f32x4 *>(reinterpret_cast<char *>(wave_base) + off), v);
  }
}
__device__ inline uint64_t wave_first(uint64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane(uint32_t(v)), hi = __builtin_amdgcn_readfirstlane(uint32_t(v >> 32));
  return (uint64_t(hi) << 32) | lo;
}

template <int CMAX, bool NLL, int NT, bool BWD, typename OFF>
__global__ __launch_bounds__(kBlock) void softmax_nd_pair_kernel(PixelGrid pg, const float *__restrict__ x,
                                                                 float *__restrict__ y,
                                                                 const uint32_t *__restrict__ cat,
                                                                 float *__restrict__ nll,
                                                                 const float *__restrict__ dy,
                                                                 float *__restrict__ dx) {
  static_assert(!BWD || NLL, "the backward pass needs the labels");
  static_assert(CMAX % 2 == 0, "two lanes share the classes");
  constexpr int H = CMAX / 2;  // classes a lane holds
  typedef std::integral_constant<int, NT & kNtLoad> LoadPolicy;
  const uint32_t block = pg.xcd ? xcd_contiguous(blockIdx.x, gridDim.x) : blockIdx.x;
  const uint32_t g = block * uint32_t(kBlock / 2) + (threadIdx.x >> 1);  // total_groups <= 2^30
  if (g >= pg.total_groups) return;  // (the lanes of a pair leave together; a wave's first lane is its lowest group)
  const uint32_t h = threadIdx.x & 1u;
  uint32_t p, n;
  pixel_decode(pg, g, 4, p, n);
  const uint64_t e = uint64_t(p) + uint64_t(pg.P) * pg.C * n;  // the group's first element in plane 0 of its sample
  const uint64_t pix = uint64_t(p) + uint64_t(pg.P) * n;
  const uint64_t e_wave = wave_first(e), pix_wave = wave_first(pix);
  const OFF off_even = OFF(e - e_wave) * OFF(4);                   // byte offsets from the wave's first group
  const OFF off = off_even + OFF(h) * (OFF(pg.P) * OFF(4));        // ... in the planes this lane holds
  const OFF off_pix = OFF(pix - pix_wave) * OFF(4);
  const uint32_t last_even = (pg.C - 1u) & ~1u;
  // the labels and the upstream gradient are requested first, so that they are there when the classes are
  u32x4 lab;
  if (NLL) lab = load_stream<0>(reinterpret_cast<const u32x4 *>(reinterpret_cast<const char *>(cat + pix_wave) + off_pix));
  f32x4 d;
  if (BWD) d = load_stream<0>(reinterpret_cast<const f32x4 *>(reinterpret_cast<const char *>(dy + pix_wave) + off_pix));
  if (NLL) issue_order_fence();
  // Every slot is loaded, a slot past the last class from the last class's plane again (and set to -inf below).
  f32x4 v[H];
#pragma unroll
  for (int i = 0; i < H; ++i) {
    const uint32_t kb = uint32_t(2 * i) < last_even ? uint32_t(2 * i) : last_even;  // wave-uniform
    v[i] = load_lane_off(x + e_wave + uint64_t(pg.P) * kb, (kb + h < pg.C) ? off : off_even, LoadPolicy{});
  }
  if (NLL) arrived(lab);
  if (BWD) {
    arrived(d);
    if (pg.ignore) {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        if (lab[w] >= pg.C) d[w] = 0.0f;
      }
    }
  }
  f32x4 m = PixVec<f32x4>::splat(kNegInf);
#pragma unroll
  for (int i = 0; i < H; ++i) {
    if (uint32_t(2 * i) + h >= pg.C) v[i] = PixVec<f32x4>::splat(kNegInf);
    m = vmax(m, v[i]);
  }
  m = vmax(m, lane_swap(m, 1));
  f32x4 s = PixVec<f32x4>::splat(0.0f);
#pragma unroll
  for (int i = 0; i < H; ++i) {
    v[i] = vexp(v[i] - m);  // a slot past the last class adds exp(-inf - m) = 0
    s += v[i];
  }
  s += lane_swap(s, 1);  // a + b == b + a: both lanes hold the same sum
  const f32x4 inv = vrcp(s);
  // the slot of this lane that holds a pixel's label, or none
  u32x4 slot;
  if (NLL) {
#pragma unroll
    for (int w = 0; w < 4; ++w) slot[w] = ((lab[w] & 1u) == h) ? (lab[w] >> 1) : 0xffffffffu;
  }
  f32x4 pick = PixVec<f32x4>::splat(0.0f);
#pragma unroll
  for (int i = 0; i < H; ++i) {
    if (NLL) {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        if (slot[w] == uint32_t(i)) pick[w] = v[i][w];
      }
    }
    if (uint32_t(2 * i) + h < pg.C) store_lane_off<NT>(y + e_wave + uint64_t(pg.P) * uint32_t(2 * i), off, v[i] * inv);
  }
  if (BWD) {
#pragma unroll
    for (int i = 0; i < H; ++i) {
      const f32x4 pr = v[i] * inv;  // the stored probability
      f32x4 gr;
#pragma unroll
      for (int w = 0; w < 4; ++w) gr[w] = d[w] * (pr[w] - (slot[w] == uint32_t(i) ? 1.0f : 0.0f));
      if (uint32_t(2 * i) + h < pg.C) store_lane_off<NT>(dx + e_wave + uint64_t(pg.P) * uint32_t(2 * i), off, gr);
    }
  }
  if (NLL) {
    // one lane of the pair holds the label's exponential, the other 0: the sum hands it to both; lane 0 multiplies
    // it by the reciprocal as the stored probability was
    pick += lane_swap(pick, 1);
    if (h == 0) {
      f32x4 out;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float pr = pick[w] * inv[w];
        out[w] = lab[w] < pg.C ? -logf(pr) : (pg.ignore ? 0.0f : __builtin_nanf(""));
      }
      store_stream<0>(reinterpret_cast<f32x4 *>(reinterpret_cast<char *>(nll + pix_wave) + off_pix), out);
    }
  }
}

// any C: one pass over the classes that keeps a running maximum and a running sum of exponentials, eight planes
// requested at a time, then a normalising pass (x is read twice; the reference reads it three times).  A block of
// planes is folded into (its maximum, the sum of its exponentials about that maximum) and merged with the running
// pair by online_merge(), which also keeps -inf planes from turning into NaN.  SPLIT lanes (1 or 8) share a group
// of W pixels, lane h taking the classes h, h + SPLIT, ...: one lane per group of four pixels leaves most of the
// GPU without work when there are few pixels and many classes ([65536, 300, 3]: 192 workgroups).
template <typename V, int SPLIT>
__global__ __launch_bounds__(kBlock) void softmax_nd_stream_kernel(PixelGrid pg, const float *__restrict__ x,
                                                                   float *__restrict__ y) {
  constexpr int W = PixVec<V>::W;
  constexpr int U = 8;
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;  // 64-bit: index + stride can pass 2^32
  const uint64_t total = uint64_t(pg.total_groups) * SPLIT;
  for (uint64_t t = uint64_t(pg.xcd ? xcd_contiguous(blockIdx.x, gridDim.x) : blockIdx.x) * kBlock + threadIdx.x; t < total; t += stride) {
    // the lanes of a group are neighbours, so they always run, and leave the loop, together
    const uint32_t g = uint32_t(t / SPLIT), h = uint32_t(t % SPLIT);
    uint32_t p, n;
    pixel_decode(pg, g, W, p, n);  // g < total_groups, which fits 32 bits
    const size_t base = size_t(p) + size_t(pg.P) * pg.C * n;
    V m = PixVec<V>::splat(kNegInf);
    V s = PixVec<V>::splat(0.0f);
    auto merge = [&](V bm, V bs) {
#pragma unroll
      for (int w = 0; w < W; ++w) {
        float mw = lane_get<V>(m, w), sw = lane_get<V>(s, w);
        online_merge(mw, sw, lane_get<V>(bm, w), lane_get<V>(bs, w));
        lane_set<V>(m, w, mw);
        lane_set<V>(s, w, sw);
      }
    };
    for (uint32_t k0 = h; k0 < pg.C; k0 += uint32_t(U * SPLIT)) {
      V v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {  // a slot past the last class reads the last class again and is set to -inf
        const uint32_t k = k0 + uint32_t(u * SPLIT);
        v[u] = load_stream<0>(reinterpret_cast<const V *>(x + base + size_t(pg.P) * (k < pg.C ? k : pg.C - 1u)));
      }
      V bm = PixVec<V>::splat(kNegInf);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (k0 + uint32_t(u * SPLIT) >= pg.C) v[u] = PixVec<V>::splat(kNegInf);
        bm = vmax(bm, v[u]);
      }
      V bs = PixVec<V>::splat(0.0f);
#pragma unroll
      for (int u = 0; u < U; ++u) bs += vexp(v[u] - bm);
#pragma unroll
      for (int w = 0; w < W; ++w) {
        if (lane_get<V>(bm, w) == kNegInf) {
          // a block of -inf planes has seen nothing: its sum, exp(-inf - -inf) = NaN, is not a sum.  A NaN among
          // them (which the maximum ignores) still has to reach the pixel's sum.
          bool nan = false;
#pragma unroll
          for (int u = 0; u < U; ++u) nan |= lane_get<V>(v[u], w) != lane_get<V>(v[u], w);
          lane_set<V>(bs, w, nan ? __builtin_nanf("") : 0.0f);
        }
      }
      merge(bm, bs);
    }
    // the lanes of the group exchange their pairs: after the last step every lane holds the same maximum, and
    // the same sum (a + b == b + a at every step)
#pragma unroll
    for (int off = 1; off < SPLIT; off <<= 1) {
      const V m2 = lane_swap(m, off), s2 = lane_swap(s, off);
      merge(m2, s2);
    }
    const V inv = vrcp(s);
    for (uint32_t k0 = h; k0 < pg.C; k0 += uint32_t(U * SPLIT)) {
      V v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t k = k0 + uint32_t(u * SPLIT);
        v[u] = load_stream<0>(reinterpret_cast<const V *>(x + base + size_t(pg.P) * (k < pg.C ? k : pg.C - 1u)));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t k = k0 + uint32_t(u * SPLIT);
        if (k < pg.C) store_stream<0>(reinterpret_cast<V *>(y + base + size_t(pg.P) * k), V(vexp(v[u] - m) * inv));
      }
    }
  }
}

// softmax.cu:278-298: per-pixel gather.  A thread takes W consecutive pixels:
// one 16-byte label load, W independent gathers in flight, one 16-byte store.
template <typename V>
__global__ __launch_bounds__(kBlock) void softmax_nd_cat_nll_kernel(PixelGrid pg, const float *__restrict__ prob,
                                                                    const uint32_t *__restrict__ cat,
                                                                    float *__restrict__ nll) {
  constexpr int W = PixVec<V>::W;
  typedef typename PixVec<V>::U U;
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;  // 64-bit: index + stride can pass 2^32
  for (uint64_t g = uint64_t(pg.xcd ? xcd_contiguous(blockIdx.x, gridDim.x) : blockIdx.x) * kBlock + threadIdx.x; g < pg.total_groups; g += stride) {
    uint32_t p, n;
    pixel_decode(pg, uint32_t(g), W, p, n);  // g < total_groups, which fits 32 bits
    const size_t pix = size_t(p) + size_t(pg.P) * n;
    const size_t base = size_t(p) + size_t(pg.P) * pg.C * n;
    const U lab = load_stream<0>(reinterpret_cast<const U *>(cat + pix));
    float pr[W];
#pragma unroll
    for (int w = 0; w < W; ++w) {
      const uint32_t k = lane_get_u(lab, w);
      pr[w] = (k < pg.C) ? prob[base + size_t(w) + size_t(pg.P) * k] : 0.0f;
    }
    V out;
#pragma unroll
    for (int w = 0; w < W; ++w) {
      lane_set<V>(out, w, lane_get_u(lab, w) < pg.C ? -logf(pr[w]) : (pg.ignore ? 0.0f : __builtin_nanf("")));
    }
    store_stream<0>(reinterpret_cast<V *>(nll + pix), out);
  }
}

// softmax.cu:315-334: dx[p,k,n] (=|+=) dy[p,n] * (prob - float(label[p,n]==k)).
// A thread reads dy and the label of its pixels once and walks the classes.
template <typename V, bool ACC, int NT>
__global__ __launch_bounds__(kBlock) void softmax_nd_cat_nll_bwd_kernel(PixelGrid pg,
                                                                        const float *__restrict__ dy,
                                                                        const float *__restrict__ prob,
                                                                        const uint32_t *__restrict__ cat,
                                                                        float *dx, uint32_t chunk) {
  constexpr int W = PixVec<V>::W;
  typedef typename PixVec<V>::U U;
  // blockIdx.y picks a run of `chunk` classes (a multiple of the four that are walked together)
  const uint32_t k_first = blockIdx.y * chunk;
  const uint32_t k_end = k_first + chunk < pg.C ? k_first + chunk : pg.C;
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;  // 64-bit: index + stride can pass 2^32
  for (uint64_t g = uint64_t(pg.xcd ? xcd_contiguous(blockIdx.x, gridDim.x) : blockIdx.x) * kBlock + threadIdx.x; g < pg.total_groups; g += stride) {
    uint32_t p, n;
    pixel_decode(pg, uint32_t(g), W, p, n);  // g < total_groups, which fits 32 bits
    const size_t pix = size_t(p) + size_t(pg.P) * n;
    const size_t base = size_t(p) + size_t(pg.P) * pg.C * n;
    V d = load_stream<0>(reinterpret_cast<const V *>(dy + pix));
    const U lab = load_stream<0>(reinterpret_cast<const U *>(cat + pix));
    if (pg.ignore) {
#pragma unroll
      for (int w = 0; w < W; ++w) {
        if (lane_get_u(lab, w) >= pg.C) lane_set<V>(d, w, 0.0f);
      }
    }
    // Four planes are requested together (a slot past the last class reads the last class again), then written:
    // the streaming store is an ordering point for the compiler, so a plane-by-plane loop keeps one load in flight.
    constexpr int B = 4;
    V pr[B], old[B];
    auto request = [&](uint32_t k0) {
#pragma unroll
      for (int u = 0; u < B; ++u) {
        const uint32_t k = k0 + uint32_t(u) < k_end ? k0 + uint32_t(u) : k_end - 1u;
        const size_t off = base + size_t(pg.P) * k;
        pr[u] = load_stream<NT>(reinterpret_cast<const V *>(prob + off));
        if (ACC) old[u] = load_stream<NT>(reinterpret_cast<const V *>(dx + off));
      }
    };
    auto write = [&](uint32_t k0) {
#pragma unroll
      for (int u = 0; u < B; ++u) {
        const uint32_t k = k0 + uint32_t(u);
        if (k < k_end) {
          V r;
#pragma unroll
          for (int w = 0; w < W; ++w) {
            const float t = lane_get<V>(pr[u], w) - float(lane_get_u(lab, w) == k);
            lane_set<V>(r, w, ACC ? fmaf(lane_get<V>(d, w), t, lane_get<V>(old[u], w)) : lane_get<V>(d, w) * t);
          }
          store_stream<NT>(reinterpret_cast<V *>(dx + base + size_t(pg.P) * k), r);
        }
      }
    };
    request(k_first);
    arrived(d);  // dy and the labels were requested first: known to be there before the first store is issued
    arrived(lab);
    write(k_first);
    for (uint32_t k0 = k_first + uint32_t(B); k0 < k_end; k0 += uint32_t(B)) {
      request(k0);
      write(k0);
    }
  }
}

PixelGrid make_pixel_grid(uint32_t P, uint32_t C, uint32_t N, int W, bool ignore = false) {
  PixelGrid pg;
  pg.ignore = ignore ? 1u : 0u;
  pg.xcd = 0u;
  pg.P = P;
  pg.C = C;
  pg.N = N;
  const uint32_t gps = (P + uint32_t(W) - 1u) / uint32_t(W);
  pg.total_groups = gps * N;
  pg.div_gps = FastDiv(gps ? gps : 1);
  return pg;
}

// one pixel group per thread: the hardware dispatcher walks the array in order
uint32_t pixel_blocks(uint32_t total_groups) { return stream_grid(total_groups, 1); }

// Whether the byte offsets of a wave's 32 pixel groups from its first group fit 32 bits in every plane the wave
// touches: 32 groups of 16 bytes, one plane's pitch for the odd lane, and a sample's pitch for every sample
// boundary the wave crosses (at most 128 / P + 1 of them).
bool nd_pair_offsets_fit(uint32_t P, uint32_t C) {
  const uint64_t crossings = 128u / P + 1u;
  return (512u + uint64_t(P) * 4u + crossings * uint64_t(P) * C * 4u) < (uint64_t(1) << 32);
}

// C <= 32, or C <= 256 in the 16-byte form, which runs two, four or eight lanes per pixel group.
template <typename V, bool NLL, int NT, bool BWD = false>
void launch_softmax_nd_reg_nt(uint32_t P, uint32_t C, uint32_t N, const float *x, float *y, const uint32_t *cat,
                              float *nll, hipStream_t s, const float *dy = nullptr, float *dx = nullptr,
                              bool ignore = false) {
  // (the same lanes per group in every variant: the order of a pixel's sum, hence the bits of p, depends on it)
  PixelGrid pg = make_pixel_grid(P, C, N, PixVec<V>::W, ignore);
  // (planes that are not whole 16-byte groups: neighbouring blocks, which write parts of the same lines, on one XCD:
  // [4225, 19] 4.9 -> 5.2 TB/s, [1025, 4] 5.3 -> 5.8, [89401, 2] 5.1 -> 5.9; [65535, 32] loses, 4.7 -> 4.3)
  pg.xcd = ((tuning().nd_xcd_mask & 1) || P % uint32_t(PixVec<V>::W) != 0) ? 1u : 0u;
  if constexpr (PixVec<V>::W == 4) {
    // more classes: eight lanes per pixel group, 8, 16 or 32 sixteen-byte values per lane
    if (C > 192) {
      softmax_nd_reg_kernel<256, V, NLL, NT, 8, BWD>
          <<<stream_grid(uint64_t(pg.total_groups) * 8, 1), kBlock, 0, s>>>(pg, x, y, cat, nll, dy, dx);
      return;
    } else if (C > 128) {
      softmax_nd_reg_kernel<192, V, NLL, NT, 8, BWD>
          <<<stream_grid(uint64_t(pg.total_groups) * 8, 1), kBlock, 0, s>>>(pg, x, y, cat, nll, dy, dx);
      return;
    } else if (C > 64) {
      softmax_nd_reg_kernel<128, V, NLL, NT, 8, BWD>
          <<<stream_grid(uint64_t(pg.total_groups) * 8, 1), kBlock, 0, s>>>(pg, x, y, cat, nll, dy, dx);
      return;
    } else if (C > 32) {
      // (eight lanes of 8 values, 106 to 123 registers, rather than four lanes of 16, 164 to 195)
      softmax_nd_reg_kernel<64, V, NLL, NT, 8, BWD>
          <<<stream_grid(uint64_t(pg.total_groups) * 8, 1), kBlock, 0, s>>>(pg, x, y, cat, nll, dy, dx);
      return;
    }
  }
  if constexpr (PixVec<V>::W == 4) {
    // two lanes per pixel group: the form with wave-uniform plane addresses, one group per lane pair
    const uint32_t pair_blocks = uint32_t((uint64_t(pg.total_groups) * 2 + kBlock - 1) / kBlock);
    auto pairs = [&](auto cmax, auto off) {
      typedef decltype(off) OFF;
      // Five workgroups per CU instead of the eight the registers allow, for 17 to 24 classes without the backward
      // pass: the forward kernel is 2-3 % faster with fewer plane-strided runs in flight ([512K, 19, 8]: 109.5 ->
      // 106.3 us; with the backward pass 174 us either way up to eight, 177 at four or five).  The cap is an LDS
      // allocation that the kernel does not touch.
      const size_t unused_lds = (!BWD && decltype(cmax)::value >= 20 && decltype(cmax)::value <= 24)
                                    ? size_t(tuning().nd_pair_ballast) * 1024 : 0;
      softmax_nd_pair_kernel<decltype(cmax)::value, NLL, NT, BWD, OFF><<<pair_blocks, kBlock, unused_lds, s>>>(pg, x, y, cat, nll, dy, dx);
    };
    auto pairs_of = [&](auto cmax) {
      if (nd_pair_offsets_fit(P, C)) {
        pairs(cmax, uint32_t(0));
      } else {
        pairs(cmax, uint64_t(0));
      }
    };
    if (C <= 2) {  // (one class per lane: with room for two, a lane would fetch its plane twice)
      pairs_of(std::integral_constant<int, 2>{});
    } else if (C <= 4) {
      pairs_of(std::integral_constant<int, 4>{});
    } else if (C <= 8) {
      pairs_of(std::integral_constant<int, 8>{});
    } else if (C <= 16) {
      pairs_of(std::integral_constant<int, 16>{});
    } else if (C <= 20) {  // 19 / 20 classes are common label sets
      pairs_of(std::integral_constant<int, 20>{});
    } else if (C <= 24) {
      pairs_of(std::integral_constant<int, 24>{});
    } else {
      pairs_of(std::integral_constant<int, 32>{});
    }
  } else {
    // one pixel per thread (planes that are not whole 16-byte groups)
    const uint32_t blocks = stream_grid(pg.total_groups, 1);
    if (C <= 4) {
      softmax_nd_reg_kernel<4, V, NLL, NT, 1, BWD><<<blocks, kBlock, 0, s>>>(pg, x, y, cat, nll, dy, dx);
    } else if (C <= 8) {
      softmax_nd_reg_kernel<8, V, NLL, NT, 1, BWD><<<blocks, kBlock, 0, s>>>(pg, x, y, cat, nll, dy, dx);
    } else if (C <= 16) {
      softmax_nd_reg_kernel<16, V, NLL, NT, 1, BWD><<<blocks, kBlock, 0, s>>>(pg, x, y, cat, nll, dy, dx);
    } else if (C <= 20) {  // 19 / 20 classes are common label sets
      softmax_nd_reg_kernel<20, V, NLL, NT, 1, BWD><<<blocks, kBlock, 0, s>>>(pg, x, y, cat, nll, dy, dx);
    } else if (C <= 24) {
      softmax_nd_reg_kernel<24, V, NLL, NT, 1, BWD><<<blocks, kBlock, 0, s>>>(pg, x, y, cat, nll, dy, dx);
    } else {
      softmax_nd_reg_kernel<32, V, NLL, NT, 1, BWD><<<blocks, kBlock, 0, s>>>(pg, x, y, cat, nll, dy, dx);
    }
  }
}

template <typename V, bool NLL, bool BWD = false>
void launch_softmax_nd_reg(uint32_t P, uint32_t C, uint32_t N, const float *x, float *y, const uint32_t *cat,
                           float *nll, hipStream_t s, const float *dy = nullptr, float *dx = nullptr) {
  // the input is streamed; the probabilities are read again by the NLL gather and the backward pass, so they
  // keep the default policy unless they are far larger than the last-level cache
  const size_t bytes = size_t(P) * C * N * sizeof(float);
  if (PixVec<V>::W == 4) {
    // (streaming stores only where every plane of the outputs starts on a 64-byte boundary)
    const int nt = (P % 16u == 0) ? policy_for_outputs(stream_policy(bytes, tuning().nontemporal), y, dx) : 0;
    with_stream_policy(nt, [&](auto policy) {
      launch_softmax_nd_reg_nt<V, NLL, decltype(policy)::value, BWD>(P, C, N, x, y, cat, nll, s, dy, dx);
    });
  } else {
    launch_softmax_nd_reg_nt<V, NLL, 0, BWD>(P, C, N, x, y, cat, nll, s, dy, dx);
  }
}

template <typename V>
void launch_softmax_nd_typed(uint32_t P, uint32_t C, uint32_t N, const float *x, float *y, hipStream_t s) {
  if (C <= 32 || (PixVec<V>::W == 4 && C <= 256)) {
    launch_softmax_nd_reg<V, false>(P, C, N, x, y, nullptr, nullptr, s);
  } else {
    const PixelGrid pg = make_pixel_grid(P, C, N, PixVec<V>::W);
    // Groups of four pixels: eight lanes per group, which is faster however many groups there are ([65536, 300, 3]
    // 3.3 TB/s against 2.3, [4096, 1000, 16] 3.3 against 0.9).  Single pixels: one lane each, so that a wave's
    // load still covers 256 contiguous bytes ([65535, 300, 3] 2.9 TB/s against 1.8 with eight lanes per pixel).
    if (PixVec<V>::W == 4) {
      softmax_nd_stream_kernel<V, 8><<<stream_grid(uint64_t(pg.total_groups) * 8, 1), kBlock, 0, s>>>(pg, x, y);
    } else {
      softmax_nd_stream_kernel<V, 1><<<pixel_blocks(pg.total_groups), kBlock, 0, s>>>(pg, x, y);
    }
  }
}

// Short planes that are not whole 64-byte pieces (P < 1024, P % 16 != 0), up to 64 classes, samples of at most
// 32 KB: a workgroup copies SB whole samples (SB * P * C contiguous floats, 16 KB where several fit) to LDS as they
// lie in memory, 16 bytes per lane, one thread per pixel walks its classes there (consecutive threads take
// consecutive pixels: consecutive banks), and the tile goes back the same way; with a gradient to write, the tile
// is turned into dy * (p - onehot) in place and goes out once more.  Every global access is full-width whatever P
// is, where the register kernels read a [196, C] sample plane by plane in 784-byte pieces: [196, 19] 4.2 -> 5.0
// TB/s, [196, 32] 3.5 -> 5.6, [49, 19] 4.4 -> 5.0, [4, 19] 1.4 -> 5.4.  (Planes of whole 64-byte pieces are as
// fast or faster through the register kernels: [16, 10] 6.0 TB/s against 5.5, [784, 4] 6.1 against 5.7; so are
// pixels of more than 64 classes, which leave most of a tile's threads idle: [4, 512] 3.0 against 1.0.)
// A pixel's sum starts at class (sample's place in the tile) mod C and wraps round, so that samples whose size is
// a multiple of the 32 banks do not all meet in the same banks; the order of a pixel's sum therefore depends on
// the shape and on the sample number, and on nothing else.  All entry points (plain, with the label gather, with
// the backward pass) run this kernel for these shapes, whatever the alignment of their arrays: their
// probabilities agree to the bit.
// Samples of more than 32 classes and up to 63 KB also have a tile to themselves where the planes are not whole
// 32-byte pieces or too long for several threads per pixel ([196, 42] 3.8 -> 4.5 TB/s, [196, 70] 2.3 -> 3.4,
// [100, 100] 2.7 -> 3.4; with few classes such samples are faster through the register kernels, [900, 12] 4.9
// against 3.7, and short planes with several threads per pixel through the column tiles, [36, 128] 5.6 against 3.3).
constexpr uint32_t kNdTileFloats = 4096;       // samples are gathered into tiles of 16 KB
constexpr uint32_t kNdTileMaxSample = 8192;    // a larger sample has a tile to itself, up to 32 KB
constexpr uint32_t kNdTileBigSample = 16128;   // ... and up to 63 KB from 33 classes on, where nothing else fits
bool nd_tile_fits(uint32_t P, uint32_t C);

struct ColReg {  // the tiling of softmax_nd_colreg_kernel, further down
  uint32_t ns, Gt, PH, tiles, xcd;
  bool fits;
};
ColReg nd_col_reg(uint32_t P, uint32_t C);

template <bool NLL, bool BWD, int NT>
__global__ __launch_bounds__(kBlock) void softmax_nd_tile_kernel(uint32_t P, uint32_t C, uint32_t N, uint32_t SB,
                                                                 FastDiv div_p, FastDiv div_c, int vec, uint32_t ignore,
                                                                 const float *__restrict__ x, float *__restrict__ y,
                                                                 const uint32_t *__restrict__ cat,
                                                                 float *__restrict__ nll,
                                                                 const float *__restrict__ dy,
                                                                 float *__restrict__ dx) {
  extern __shared__ __align__(16) float tile[];  // SB * P * C floats, at most kNdTileBigSample
  f32x4 *tile4 = reinterpret_cast<f32x4 *>(tile);
  const uint32_t slab = P * C;
  for (uint64_t n0 = uint64_t(blockIdx.x) * SB; n0 < N; n0 += uint64_t(gridDim.x) * SB) {
    const uint32_t samples = (N - n0 < uint64_t(SB)) ? uint32_t(N - n0) : SB;
    const uint32_t n = samples * slab;
    const uint32_t n4 = vec ? n / 4u : 0u;  // (16-byte copies; what is left of the tile goes element by element)
    const float *xt = x + n0 * slab;
    float *yt = y + n0 * slab;
    // eight groups per thread are requested before the first is written to LDS (a slot past the tile's end reads
    // its last group again and is dropped)
    // A wave's step covers whole 128-byte lines of the array: the groups are taken `ax` places later, ax = the
    // tile's distance in groups from the line before it, so that the first wave's first step is the short one
    // (a sample of 19 planes of 196 pixels starts anywhere in a line; [196, 19] 4.9 -> 5.2 TB/s, [49, 19] 4.8 -> 5.3).
    // (a tile of fewer than four floats -- a last tile of one sample of a 2- or 3-pixel, one-class array -- has no
    // group to clamp to: it takes the element loop below alone)
    const uint32_t ax = vec ? uint32_t((reinterpret_cast<uintptr_t>(xt) >> 4) & 7u) : 0u;
    for (uint32_t g0 = 0; n4 != 0u && g0 < n4 + ax; g0 += 8u * kBlock) {
      f32x4 in[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t slot = g0 + threadIdx.x + uint32_t(i) * kBlock;
        const uint32_t g = slot >= ax ? slot - ax : 0u;
        in[i] = load_stream<NT>(reinterpret_cast<const f32x4 *>(xt) + (g < n4 ? g : n4 - 1u));
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t slot = g0 + threadIdx.x + uint32_t(i) * kBlock;
        if (slot >= ax && slot - ax < n4) tile4[slot - ax] = in[i];
      }
    }
    for (uint32_t e = n4 * 4u + threadIdx.x; e < n; e += kBlock) tile[e] = xt[e];
    __syncthreads();
    const uint32_t pixels = samples * P;
    const size_t pix0 = size_t(n0) * P;
    for (uint32_t q = threadIdx.x; q < pixels; q += kBlock) {
      uint32_t sb, pp;
      div_p.divmod(q, sb, pp);
      // the label is requested before the walk, so that it is there after it
      uint32_t label = 0u;
      if (NLL) label = cat[pix0 + q];
      float *col = tile + sb * slab + pp;  // class k of this pixel is col[k * P]
      const uint32_t first = sb - div_c.div(sb) * C;
      float m = kNegInf;
#pragma unroll 4
      for (uint32_t k = 0; k < C; ++k) m = fmaxf(m, col[k * P]);
      float sum = 0.0f;  // classes first .. C - 1, then 0 .. first - 1
#pragma unroll 4
      for (uint32_t k = first; k < C; ++k) {
        const float e = exp_nonpos(col[k * P] - m);
        col[k * P] = e;
        sum += e;
      }
#pragma unroll 4
      for (uint32_t k = 0; k < first; ++k) {
        const float e = exp_nonpos(col[k * P] - m);
        col[k * P] = e;
        sum += e;
      }
      const float inv = 1.0f / sum;  // one correctly rounded reciprocal per pixel
#pragma unroll 4
      for (uint32_t k = 0; k < C; ++k) col[k * P] *= inv;
      if (NLL) {
        // -log of the stored probability of the label; NaN (0 with `ignore`) when the label is out of range
        nll[pix0 + q] = label < C ? -logf(col[label * P]) : (ignore ? 0.0f : __builtin_nanf(""));
      }
    }
    __syncthreads();
    const uint32_t ay = vec ? uint32_t((reinterpret_cast<uintptr_t>(yt) >> 4) & 7u) : 0u;
    for (uint32_t slot = threadIdx.x; slot < n4 + ay; slot += kBlock) {
      if (slot >= ay) store_stream<NT>(reinterpret_cast<f32x4 *>(yt) + (slot - ay), tile4[slot - ay]);
    }
    for (uint32_t e = n4 * 4u + threadIdx.x; e < n; e += kBlock) yt[e] = tile[e];
    __syncthreads();  // the tile is overwritten below, or by the next pass
    if (BWD) {
      for (uint32_t q = threadIdx.x; q < pixels; q += kBlock) {
        uint32_t sb, pp;
        div_p.divmod(q, sb, pp);
        const uint32_t label = cat[pix0 + q];
        float d = dy[pix0 + q];
        if (ignore && label >= C) d = 0.0f;
        float *col = tile + sb * slab + pp;
#pragma unroll 4
        for (uint32_t k = 0; k < C; ++k) col[k * P] = d * (col[k * P] - float(label == k));
      }
      __syncthreads();
      float *dt = dx + n0 * slab;
      const uint32_t ad = vec ? uint32_t((reinterpret_cast<uintptr_t>(dt) >> 4) & 7u) : 0u;
      for (uint32_t slot = threadIdx.x; slot < n4 + ad; slot += kBlock) {
        if (slot >= ad) store_stream<NT>(reinterpret_cast<f32x4 *>(dt) + (slot - ad), tile4[slot - ad]);
      }
      for (uint32_t e = n4 * 4u + threadIdx.x; e < n; e += kBlock) dt[e] = tile[e];
      __syncthreads();
    }
  }
}

template <bool NLL, bool BWD>
void launch_softmax_nd_tile(uint32_t P, uint32_t C, uint32_t N, const float *x, float *y, const uint32_t *cat,
                            float *nll, const float *dy, float *dx, bool ignore, hipStream_t s) {
  const uint32_t slab = P * C;
  // as many samples as fit, but no more than leaves every CU two workgroups; from four on a multiple of four,
  // so that every tile starts a whole number of 16-byte groups into the array
  uint32_t SB = kNdTileFloats / slab;
  const uint32_t spread = (N + 2u * uint32_t(device_cu_count()) - 1u) / (2u * uint32_t(device_cu_count()));
  if (SB > spread) SB = spread;
  if (SB >= 4u) SB &= ~3u;
  if (SB == 0u) SB = 1u;
  uint32_t blocks = (N + SB - 1u) / SB;
  const uint32_t max_blocks = 1u << 24;
  if (blocks > max_blocks) blocks = max_blocks;
  // 16-byte copies between the arrays and the tile wherever the tiles start (4-byte-aligned accesses; with 4-byte
  // copies for tiles that do not start a whole number of groups into the array, [169, 19] ran at 3.5 TB/s)
  const int vec = 1;
  // streaming stores where every tile starts a whole number of 16-byte groups into the array: the copy steps of a
  // wave then cover whole lines of the array wherever the tile starts ([196, 19] 5.5 TB/s with ordinary stores, 6.0)
  const bool whole_pieces = (uint64_t(SB) * slab) % 4u == 0 || N <= SB;
  const size_t lds_bytes = size_t(SB) * slab * sizeof(float);
  const FastDiv div_p(P), div_c(C);
  // logits in, probabilities (and the gradient) out: all streamed
  const int nt = whole_pieces ? policy_for_outputs(stream_policy(size_t(slab) * N * sizeof(float), tuning().nontemporal), y, dx) : 0;
  with_stream_policy(nt, [&](auto policy) {
    softmax_nd_tile_kernel<NLL, BWD, decltype(policy)::value>
        <<<blocks, kBlock, lds_bytes, s>>>(P, C, N, SB, div_p, div_c, vec, ignore ? 1u : 0u, x, y, cat, nll, dy, dx);
  });
}

// More classes than the register kernels hold well (from 193 on; from 65 on for planes shorter than 1024 pixels),
// 16-byte accesses: a workgroup takes a tile of TP consecutive pixels of one sample with all their classes -- C runs
// of TP floats, one per plane, 32 KB together (up to 59 KB where that is what 32 pixels, or 16 of a short plane,
// take) -- into LDS, row k of the tile holding plane k's run, 16 bytes per lane both ways.  L = 256 / TP threads
// share a pixel: thread (j, l) walks classes l, l + L, ... of pixel j (consecutive threads take consecutive pixels:
// consecutive banks); the L maxima and the L sums of a pixel meet through LDS.  x is read once, where the streaming
// kernel reads it twice, and a lane holds nothing but its running values, where the register kernel holds 32 values
// of 16 bytes: [65536, 200] 4.1 -> 4.6 TB/s, [65536, 300] 3.4 -> 3.9, [4096, 300] 3.3 -> 4.4, [1024, 256] 4.3 -> 5.2,
// [784, 100] 3.2 -> 5.2, [64, 100] 3.3 -> 5.6, [64, 300] 3.2 -> 4.4, [16, 256] 4.6 -> 5.8.  (From 65 to 192 classes on long planes the register
// kernels are faster, 5.0-5.2 against 4.5-5.0.)  Long planes are cut into runs of whole 128-byte lines, short ones
// into tiles of about the same width.  A pixel's sum is the sum of its L partial sums, each added in class order:
// the order depends on the shape and on nothing else.  Every entry point (plain, with the label gather, with the
// backward pass) runs this kernel for these shapes.
constexpr uint32_t kColTileFloats = 8192;      // the tile a workgroup aims for: four workgroups per CU
constexpr uint32_t kColTileMaxFloats = 15104;  // the largest tile, 59 KB, beside 5 KB of per-pixel arrays

struct ColTile {
  uint32_t TP;  // pixels per tile: a multiple of 4, 16 to 256
  uint32_t L;   // threads per pixel
  uint32_t tiles_per_sample;
  bool fits;
};

ColTile nd_col_tile(uint32_t P, uint32_t C) {
  ColTile ct = {0, 0, 0, false};
  if (P % 4u != 0 || P < 16 || C < (P < 1024 ? 65u : 193u)) return ct;
  uint32_t TP = (kColTileFloats / C) & ~3u;
  if (TP < 32) TP = (kColTileMaxFloats / C) & ~3u;  // many classes: the largest tile
  if (TP < 16) return ct;
  if (TP > 256) TP = 256;
  if (TP >= P) {
    TP = P;
  } else if (P >= 1024) {
    if (TP < 32) return ct;
    TP &= ~31u;  // runs of whole 128-byte lines
  } else {
    // Short planes: tiles of about the same width.  Planes that are not whole 32-byte pieces are left to the other
    // kernels unless a tile holds a whole plane: their runs start anywhere in a piece, and cut runs then share
    // pieces with their neighbours ([196, 128] 2.5 TB/s against 3.5).
    // (from 256 pixels on they take the column tiles up to 128 classes, with ordinary stores, which the L2 merges:
    // [676, 100] 3.1 -> 3.9 TB/s, [900, 65] 2.6 -> 4.0 against one pixel per thread; beyond 128 classes the kernels with
    // eight lanes per pixel group are as fast or faster, [900, 150] 4.1 against 3.6)
    if (P % 8u != 0 && (P < 256u || C > 128u)) return ct;
    const uint32_t tiles = (P + TP - 1) / TP;
    const uint32_t width = (P + tiles - 1) / tiles;
    if (P % 16u == 0) {
      // runs of whole 64-byte pieces: a run that ends inside a piece shares it with the next tile's, and both
      // write a part of it ([400, 128] in runs of 240 bytes 2.9 TB/s, [576, 200] in runs of 160 bytes 2.9)
      TP = (width + 15u) & ~15u;
      if (uint64_t(TP) * C > kColTileMaxFloats) TP -= 16u;
      if (TP < 16u) return ct;
    } else {
      TP = (width + 3u) & ~3u;
    }
  }
  ct.TP = TP;
  ct.L = 256u / TP;
  ct.tiles_per_sample = (P + TP - 1) / TP;
  ct.fits = true;
  return ct;
}

bool nd_tile_fits(uint32_t P, uint32_t C) {
  if (!(P > 1 && P < 1024 && P % 16u != 0)) return false;
  const uint64_t sample = uint64_t(P) * C;
  if (C <= 64 && sample <= kNdTileMaxSample) return true;
  if (C > 32 && sample <= kNdTileBigSample) {
    // (from 128 pixels on, column tiles in registers: [169, 64] 4.3 TB/s through a tile of one sample, 5.5 through them; [225, 64] 3.8 -> 5.4)
    if (nd_col_reg(P, C).fits) return false;
    const ColTile ct = nd_col_tile(P, C);
    return !(ct.fits && ct.L >= 2);  // several threads per pixel over whole planes are faster
  }
  return false;
}

template <bool NLL, bool BWD, int NT>
__global__ __launch_bounds__(kBlock) void softmax_nd_coltile_kernel(uint32_t P, uint32_t C, uint32_t TP, uint32_t L,
                                                                    uint32_t total_tiles, FastDiv div_tps,
                                                                    FastDiv div_tp, uint32_t ignore, uint32_t xcd,
                                                                    const float *__restrict__ x, float *__restrict__ y,
                                                                    const uint32_t *__restrict__ cat,
                                                                    float *__restrict__ nll,
                                                                    const float *__restrict__ dy,
                                                                    float *__restrict__ dx) {
  extern __shared__ __align__(16) float smem[];
  float *tile = smem;                                          // C rows of TP floats
  float *part_max = tile + C * TP;                             // [L][TP]
  float *part_sum = part_max + kBlock;                         // [L][TP]
  float *inv = part_sum + kBlock;                              // [TP]
  uint32_t *labs = reinterpret_cast<uint32_t *>(inv + kBlock);  // [TP]
  float *dys = reinterpret_cast<float *>(labs + kBlock);       // [TP]
  f32x4 *tile4 = reinterpret_cast<f32x4 *>(tile);
  const uint32_t row4 = TP / 4u;  // 16-byte groups per tile row
  uint32_t l, j;                  // this thread's place in the pixel phases
  div_tp.divmod(threadIdx.x, l, j);
  // One tile per workgroup (a workgroup that walked several tiles, with the next tile's loads requested before the
  // current tile's pixel phases, measured slower: [784, 100] 4.1 TB/s against 5.3).  With `xcd` (long planes),
  // neighbouring tiles run on the same XCD: [1024, 256] 4.7 -> 5.2 TB/s, [4096, 150] 4.7 -> 5.1; on short planes
  // it loses ([196, 100] 3.5 -> 3.2, [16, 256] 5.8 -> 5.5).
  for (uint32_t b0 = blockIdx.x; b0 < total_tiles; b0 += gridDim.x) {
    const uint32_t b = (xcd && gridDim.x == total_tiles) ? xcd_contiguous(b0, total_tiles) : b0;
    uint32_t n, ti;
    div_tps.divmod(b, n, ti);
    const uint32_t p0 = ti * TP;
    const uint32_t tp = P - p0 < TP ? P - p0 : TP;  // a multiple of 4, as P and TP are
    const size_t base = size_t(P) * C * n + p0;
    const size_t pix = size_t(P) * n + p0;
    if (NLL && threadIdx.x < tp) {
      const uint32_t label = cat[pix + threadIdx.x];
      labs[threadIdx.x] = label;
      if (BWD) dys[threadIdx.x] = (ignore && label >= C) ? 0.0f : dy[pix + threadIdx.x];
    }
    // Group q of the tile is group q % ppr of plane q / ppr's run; a thread's groups are 256 apart, so (k, jj) moves
    // by (256 / ppr, 256 % ppr) with a carry.
    const uint32_t ppr = tp / 4u, groups = C * ppr;
    const uint32_t step_k = kBlock / ppr, step_j = kBlock % ppr;
    const uint32_t k_first = threadIdx.x / ppr, jj_first = threadIdx.x - k_first * ppr;
    {
      uint32_t k = k_first, jj = jj_first;
      // eight groups per thread are requested before the first is written to LDS (a slot past the tile's end reads
      // the tile's first group again and is dropped)
      for (uint32_t q0 = 0; q0 < groups; q0 += 8u * kBlock) {
        f32x4 in[8];
        uint32_t at[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const bool live = q0 + threadIdx.x + uint32_t(i) * kBlock < groups;
          at[i] = live ? k * row4 + jj : 0xffffffffu;
          in[i] = load_stream<NT>(reinterpret_cast<const f32x4 *>(x + base + (live ? size_t(P) * k + 4u * jj : 0)));
          k += step_k;
          jj += step_j;
          if (jj >= ppr) {
            jj -= ppr;
            ++k;
          }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (at[i] != 0xffffffffu) tile4[at[i]] = in[i];
        }
      }
    }
    __syncthreads();
    const bool active = l < L && j < tp;
    float m = kNegInf;
    if (active) {
#pragma unroll 4
      for (uint32_t k = l; k < C; k += L) m = fmaxf(m, tile[k * TP + j]);
      part_max[l * TP + j] = m;
    }
    __syncthreads();
    if (active) {
      for (uint32_t ll = 0; ll < L; ++ll) m = fmaxf(m, part_max[ll * TP + j]);
      float sum = 0.0f;
#pragma unroll 4
      for (uint32_t k = l; k < C; k += L) {
        const float e = exp_nonpos(tile[k * TP + j] - m);
        tile[k * TP + j] = e;
        sum += e;
      }
      part_sum[l * TP + j] = sum;
    }
    __syncthreads();
    if (threadIdx.x < tp) {
      float sum = part_sum[threadIdx.x];
      for (uint32_t ll = 1; ll < L; ++ll) sum += part_sum[ll * TP + threadIdx.x];
      const float r = 1.0f / sum;  // one correctly rounded reciprocal per pixel
      inv[threadIdx.x] = r;
      if (NLL) {
        // -log of the stored probability of the label; NaN (0 with `ignore`) when the label is out of range
        const uint32_t label = labs[threadIdx.x];
        nll[pix + threadIdx.x] =
            label < C ? -logf(tile[label * TP + threadIdx.x] * r) : (ignore ? 0.0f : __builtin_nanf(""));
      }
    }
    __syncthreads();
    {
      uint32_t k = k_first, jj = jj_first;
      for (uint32_t q = threadIdx.x; q < groups; q += kBlock) {
        const f32x4 e = tile4[k * row4 + jj];
        const f32x4 r = reinterpret_cast<const f32x4 *>(inv)[jj];
        const f32x4 pr = {e.x * r.x, e.y * r.y, e.z * r.z, e.w * r.w};
        const size_t off = base + size_t(P) * k + 4u * jj;
        store_stream<NT>(reinterpret_cast<f32x4 *>(y + off), pr);
        if (BWD) {
          const u32x4 lab = reinterpret_cast<const u32x4 *>(labs)[jj];
          const f32x4 d = reinterpret_cast<const f32x4 *>(dys)[jj];
          f32x4 gr;
#pragma unroll
          for (int w = 0; w < 4; ++w) gr[w] = d[w] * (pr[w] - float(lab[w] == k));
          store_stream<NT>(reinterpret_cast<f32x4 *>(dx + off), gr);
        }
        k += step_k;
        jj += step_j;
        if (jj >= ppr) {
          jj -= ppr;
          ++k;
        }
      }
    }
    __syncthreads();  // the next tile overwrites all of it
  }
}

template <bool NLL, bool BWD>
void launch_softmax_nd_coltile(const ColTile &ct, uint32_t P, uint32_t C, uint32_t N, const float *x, float *y,
                               const uint32_t *cat, float *nll, const float *dy, float *dx, bool ignore,
                               hipStream_t s) {
  const uint32_t total_tiles = ct.tiles_per_sample * N;  // at most len / 16
  const uint32_t max_blocks = 1u << 24;
  const uint32_t blocks = total_tiles < max_blocks ? total_tiles : max_blocks;
  const size_t lds_bytes = (size_t(C) * ct.TP + 5u * kBlock) * sizeof(float);
  const FastDiv div_tps(ct.tiles_per_sample), div_tp(ct.TP);
  const uint32_t xcd = P >= 1024 ? 1u : 0u;
  // logits in, probabilities (and the gradient) out: all streamed
  // (streaming stores only where every run of a tile is whole 64-byte pieces, or a tile holds whole samples)
  const int nt = (P % 16u == 0 || ct.TP >= P) ? policy_for_outputs(stream_policy(size_t(P) * C * N * sizeof(float), tuning().nontemporal), y, dx) : 0;
  with_stream_policy(nt, [&](auto policy) {
    softmax_nd_coltile_kernel<NLL, BWD, decltype(policy)::value><<<blocks, kBlock, lds_bytes, s>>>(
        P, C, ct.TP, ct.L, total_tiles, div_tps, div_tp, ignore ? 1u : 0u, xcd, x, y, cat, nll, dy, dx);
  });
}

// Whole samples in registers, for short planes of whole 16-byte groups with many classes: one workgroup per sample,
// whose G = P / 4 pixel groups times C classes lie contiguously in memory.  Thread t = phase * G + g holds pixel group
// g of the classes phase, phase + PH, phase + 2 PH, ... (PH = threads / G phases, at most NS classes per thread), so
// slot i of the workgroup's live threads is the contiguous run of G * PH groups that starts i * G * PH groups into
// the sample: every access is 16 bytes per lane over whole runs of the array, whatever P is, x is read once, and
// nothing but the PH partial maxima and sums of a pixel group goes through LDS.  A pixel's sum is the sum of its PH
// partial sums in phase order, each added in class order: it depends on the shape and on nothing else.
struct SampleReg {
  uint32_t threads;  // 256, 512 or 1024: the kernel's launch bound
  uint32_t ns;       // 8 or 16 slots per thread
  uint32_t G, PH;
  bool fits;
};

template <int NS, int THREADS, bool NLL, bool BWD, int NT>
__global__ __launch_bounds__(THREADS) void softmax_nd_samplereg_kernel(uint32_t P, uint32_t C, uint32_t N, uint32_t G,
                                                                      uint32_t PH, FastDiv div_g, uint32_t ignore,
                                                                      const float *__restrict__ x,
                                                                      float *__restrict__ y,
                                                                      const uint32_t *__restrict__ cat,
                                                                      float *__restrict__ nll,
                                                                      const float *__restrict__ dy,
                                                                      float *__restrict__ dx) {
  static_assert(!BWD || NLL, "the backward pass needs the labels");
  __shared__ f32x4 part_max[THREADS], part_sum[THREADS];
  const uint32_t t = threadIdx.x;
  const uint32_t live_threads = G * PH;
  const bool live = t < live_threads;
  uint32_t phase, g;
  div_g.divmod(t, phase, g);
  const size_t sample = size_t(P) * C;
  const f32x4 ninf = PixVec<f32x4>::splat(kNegInf);
  for (uint64_t n = blockIdx.x; n < N; n += gridDim.x) {
    const f32x4 *xs = reinterpret_cast<const f32x4 *>(x + n * sample);
    const size_t pix = n * P + 4u * g;
    u32x4 lab = {0u, 0u, 0u, 0u};
    f32x4 d = {0.0f, 0.0f, 0.0f, 0.0f};
    if (NLL && live) lab = load_stream<0>(reinterpret_cast<const u32x4 *>(cat + pix));
    if (BWD && live) d = load_stream<0>(reinterpret_cast<const f32x4 *>(dy + pix));
    f32x4 v[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const uint32_t c = uint32_t(i) * PH + phase;
      v[i] = (live && c < C) ? load_stream<NT>(xs + (size_t(i) * live_threads + t)) : ninf;
    }
    f32x4 m = ninf;
#pragma unroll
    for (int i = 0; i < NS; ++i) m = vmax(m, v[i]);
    if (live) part_max[t] = m;
    __syncthreads();
    if (live) {
      m = part_max[g];
      for (uint32_t ph = 1; ph < PH; ++ph) m = vmax(m, part_max[ph * G + g]);
    }
    f32x4 sum = PixVec<f32x4>::splat(0.0f);
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const uint32_t c = uint32_t(i) * PH + phase;
      v[i] = (live && c < C) ? vexp(v[i] - m) : PixVec<f32x4>::splat(0.0f);
      sum += v[i];
    }
    if (live) part_sum[t] = sum;
    __syncthreads();
    if (live) {
      sum = part_sum[g];
      for (uint32_t ph = 1; ph < PH; ++ph) sum += part_sum[ph * G + g];
      const f32x4 inv = vrcp(sum);  // one correctly rounded reciprocal per pixel
      if (BWD && ignore) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          if (lab[w] >= C) d[w] = 0.0f;
        }
      }
      f32x4 *ys = reinterpret_cast<f32x4 *>(y + n * sample);
      f32x4 *ds = BWD ? reinterpret_cast<f32x4 *>(dx + n * sample) : nullptr;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const uint32_t c = uint32_t(i) * PH + phase;
        if (c < C) {
          const f32x4 pr = v[i] * inv;
          store_stream<NT>(ys + (size_t(i) * live_threads + t), pr);
          if (NLL) {
            // -log of the stored probability, by the thread that holds the label's class
#pragma unroll
            for (int w = 0; w < 4; ++w) {
              if (lab[w] == c) nll[pix + uint32_t(w)] = -logf(pr[w]);
            }
          }
          if (BWD) {
            f32x4 gr;
#pragma unroll
            for (int w = 0; w < 4; ++w) gr[w] = d[w] * (pr[w] - float(lab[w] == c));
            store_stream<NT>(ds + (size_t(i) * live_threads + t), gr);
          }
        }
      }
      if (NLL && phase == 0u) {  // a label out of range: NaN (0 with `ignore`)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          if (lab[w] >= C) nll[pix + uint32_t(w)] = ignore ? 0.0f : __builtin_nanf("");
        }
      }
    }
    // (part_max is written again only after the barrier above, part_sum only after the next one)
  }
}

// Which form of the kernel a shape takes, if any.  Forms in the order they are tried: (threads, slots per thread)
// with the workgroups of it that fit a CU by registers -- (256, 8) eight, (256, 16) and (512, 8) four, (512, 16) and
// (1024, 8) two, (1024, 16) one.  The first form that holds the classes and keeps at least 64 KB of samples in
// flight per CU is taken (a [36, 33] sample is 4.6 KB: eight of them leave the memory system idle, 3.1 TB/s against
// 5.8 through the LDS tiles); at most 32 phases, since every thread reads all partial values of its pixel group
// ([16, 200] with 64 phases: 4.2 TB/s against 5.8).  One workgroup of 1024 threads per CU loads, reduces and stores
// in turn, 4.6-4.9 TB/s: taken only from 129 classes on, or for planes that are not whole 64-byte pieces, where the
// other kernels run at 2.6-3.9.
// Measured on 256 MB arrays, against the kernels that took these shapes before (LDS tiles, column tiles, one pixel
// per thread, eight lanes per pixel group): [196, 64] 4.7 -> 5.5 TB/s, [196, 100] 3.1 -> 5.3, [196, 150] 3.9 -> 5.1,
// [196, 200 / 256 / 300] 3.1 / 3.3 / 2.7 -> 4.6, [100, 100 ... 300] 2.6-4.0 -> 5.3-5.8, [36, 256] 2.1 -> 5.7,
// [256, 150] 3.0 -> 4.7, [400, 150] 2.6 -> 4.9, [64, 33] 4.8 -> 6.1, [400, 33] 4.6 -> 5.9; within 6 % either way at
// [64, 100], [100, 33], [196, 33], [36, 200].
SampleReg nd_sample_reg(uint32_t P, uint32_t C) {
  SampleReg sr = {0, 0, 0, 0, false};
  if (tuning().nd_sample_reg == 0) return sr;
  if (P % 4u != 0 || P < 8u || P >= 1024u || C <= 32u) return sr;  // (longer planes never hold 33 classes in a form that is taken)
  // (samples of up to 32 KB on planes of 96 pixels and more keep the LDS tile, where enough threads of a tile have a
  // pixel to walk: [196, 33] 5.9 TB/s against 5.5, [100, 48] 5.7 against 5.5)
  if (C <= 64u && P >= 96u && uint64_t(P) * C <= kNdTileMaxSample && nd_tile_fits(P, C)) return sr;
  const uint32_t G = P / 4u;
  const uint64_t sample_bytes = uint64_t(P) * C * sizeof(float);
  const uint32_t forms[6][3] = {{256, 8, 8}, {256, 16, 4}, {512, 8, 4}, {512, 16, 2}, {1024, 8, 2}, {1024, 16, 1}};
  for (const auto &f : forms) {
    uint32_t PH = f[0] / G;
    if (PH > 32u) PH = 32u;
    if (PH == 0 || uint64_t(PH) * f[1] < C) continue;
    if (f[2] * sample_bytes < (64u << 10)) return sr;  // (the later forms keep no more in flight)
    // (from 128 pixels on, tiles of the planes in registers are faster than a sample per 1024 threads: [256, 150] 4.8
    // against 5.9 TB/s, [196, 200] 4.4 against 5.2)
    if (f[0] == 1024u && nd_col_reg(P, C).fits) return sr;
    if (f[2] == 1u && C <= 128u && P % 16u == 0) return sr;  // (planes of whole 64-byte pieces: the column tiles, 5.0-5.8 TB/s)
    sr.threads = f[0];
    sr.ns = f[1];
    sr.G = G;
    sr.PH = PH;
    sr.fits = true;
    return sr;
  }
  return sr;
}

template <bool NLL, bool BWD>
void launch_softmax_nd_samplereg(const SampleReg &sr, uint32_t P, uint32_t C, uint32_t N, const float *x, float *y,
                                 const uint32_t *cat, float *nll, const float *dy, float *dx, bool ignore,
                                 hipStream_t s) {
  uint32_t max_blocks = 1u << 24;
  if (tuning().flat_wg_per_cu > 0) max_blocks = uint32_t(device_cu_count()) * uint32_t(tuning().flat_wg_per_cu);  // (the tests' way into the loop over samples)
  const uint32_t blocks = N < max_blocks ? N : max_blocks;
  const uint32_t live_threads = sr.G * sr.PH;
  const uint32_t launch_threads = (live_threads + kWave - 1u) / kWave * kWave;
  const FastDiv div_g(sr.G);
  // streaming stores only where every step of every sample starts on a 64-byte boundary
  const bool whole_pieces = (uint64_t(P) * C) % 16u == 0 && live_threads % 4u == 0;
  const int nt = whole_pieces ? policy_for_outputs(stream_policy(size_t(P) * C * N * sizeof(float), tuning().nontemporal), y, dx) : 0;
  with_stream_policy(nt, [&](auto policy) {
    constexpr int NT = decltype(policy)::value;
    auto go = [&](auto ns, auto threads) {
      softmax_nd_samplereg_kernel<decltype(ns)::value, decltype(threads)::value, NLL, BWD, NT>
          <<<blocks, launch_threads, 0, s>>>(P, C, N, sr.G, sr.PH, div_g, ignore ? 1u : 0u, x, y, cat, nll, dy, dx);
    };
    auto with_ns = [&](auto threads) {
      if (sr.ns == 8) {
        go(std::integral_constant<int, 8>{}, threads);
      } else {
        go(std::integral_constant<int, 16>{}, threads);
      }
    };
    if (sr.threads == 256) {
      with_ns(std::integral_constant<int, 256>{});
    } else if (sr.threads == 512) {
      with_ns(std::integral_constant<int, 512>{});
    } else {
      with_ns(std::integral_constant<int, 1024>{});
    }
  });
}

// Column tiles in registers, for 33 to 1024 classes on planes of 128 pixels and more: the
// kernel above with a workgroup per run of Gt pixel groups of one sample instead of per sample.  Thread t =
// phase * Gt + g holds pixel group g of the tile for the classes phase, phase + PH, ...: a wave reads, per slot, 64 / Gt
// runs of Gt * 16 bytes, one per plane, and x is read once with nothing but the partial maxima and sums in LDS (the
// LDS column tiles below move every value through LDS five times).  Against the kernels that took these shapes before
// (eight lanes per pixel group up to 256 classes, LDS column tiles, the two-pass kernel beyond), 256 MB arrays:
// [65536, 64] 5.3 -> 5.9 TB/s, [65536, 200] 4.9 -> 5.5, [65536, 256] 4.3 -> 5.4, [65536, 300] 4.3 -> 5.1,
// [65536, 512] 3.5 -> 4.9, [2048, 256] 4.7 -> 5.9, [784, 300] 3.7 -> 5.1, [256, 300] 3.5 -> 5.6; planes that are not
// whole 128-byte lines, with neighbouring tiles on one XCD so that the lines they share are fetched once:
// [900, 100] 3.9 -> 5.6, [900, 200] 3.1 -> 5.3, [1028, 64] 4.0 -> 5.6, [676, 128] 3.8 -> 5.5.
template <int NS, int THREADS, bool NLL, bool BWD, int NT>
__global__ __launch_bounds__(THREADS) void softmax_nd_colreg_kernel(uint32_t P, uint32_t C, uint32_t Gt, uint32_t PH,
                                                                   uint32_t total_tiles, FastDiv div_gt,
                                                                   FastDiv div_tiles, uint32_t ignore, uint32_t xcd,
                                                                   const float *__restrict__ x, float *__restrict__ y,
                                                                   const uint32_t *__restrict__ cat,
                                                                   float *__restrict__ nll,
                                                                   const float *__restrict__ dy,
                                                                   float *__restrict__ dx) {
  static_assert(!BWD || NLL, "the backward pass needs the labels");
  __shared__ f32x4 part_max[THREADS], part_sum[THREADS];
  const uint32_t t = threadIdx.x;
  uint32_t phase, g;
  div_gt.divmod(t, phase, g);
  const f32x4 ninf = PixVec<f32x4>::splat(kNegInf);
  for (uint32_t b0 = blockIdx.x; b0 < total_tiles; b0 += gridDim.x) {
    const uint32_t b = (xcd && gridDim.x == total_tiles) ? xcd_contiguous(b0, total_tiles) : b0;
    uint32_t n, ti;
    div_tiles.divmod(b, n, ti);
    const uint32_t P4 = (P + 3u) / 4u;  // pixel groups of a plane; the last one ends with the plane (PixelGrid)
    const uint32_t g0 = ti * Gt;
    const uint32_t gt = P4 - g0 < Gt ? P4 - g0 : Gt;
    const bool live = phase < PH && g < gt;
    uint32_t p = 4u * (g0 + g);
    if (p + 4u > P) p = P - 4u;
    const size_t first = size_t(n) * C * P + p;  // class c of this thread's pixels is c * P further
    const float *xs = x + first;
    const size_t pix = size_t(n) * P + p;
    u32x4 lab = {0u, 0u, 0u, 0u};
    f32x4 d = {0.0f, 0.0f, 0.0f, 0.0f};
    if (NLL && live) lab = load_stream<0>(reinterpret_cast<const u32x4 *>(cat + pix));
    if (BWD && live) d = load_stream<0>(reinterpret_cast<const f32x4 *>(dy + pix));
    f32x4 v[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const uint32_t c = uint32_t(i) * PH + phase;
      v[i] = (live && c < C) ? load_stream<NT>(reinterpret_cast<const f32x4 *>(xs + size_t(c) * P)) : ninf;
    }
    f32x4 m = ninf;
#pragma unroll
    for (int i = 0; i < NS; ++i) m = vmax(m, v[i]);
    if (live) part_max[t] = m;
    __syncthreads();
    if (live) {
      m = part_max[g];
      for (uint32_t ph = 1; ph < PH; ++ph) m = vmax(m, part_max[ph * Gt + g]);
    }
    f32x4 sum = PixVec<f32x4>::splat(0.0f);
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      const uint32_t c = uint32_t(i) * PH + phase;
      v[i] = (live && c < C) ? vexp(v[i] - m) : PixVec<f32x4>::splat(0.0f);
      sum += v[i];
    }
    if (live) part_sum[t] = sum;
    __syncthreads();
    if (live) {
      sum = part_sum[g];
      for (uint32_t ph = 1; ph < PH; ++ph) sum += part_sum[ph * Gt + g];
      const f32x4 inv = vrcp(sum);
      if (BWD && ignore) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          if (lab[w] >= C) d[w] = 0.0f;
        }
      }
      float *ys = y + first;
      float *ds = BWD ? dx + first : nullptr;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const uint32_t c = uint32_t(i) * PH + phase;
        if (c < C) {
          const f32x4 pr = v[i] * inv;
          store_stream<NT>(reinterpret_cast<f32x4 *>(ys + size_t(c) * P), pr);
          if (NLL) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
              if (lab[w] == c) nll[pix + uint32_t(w)] = -logf(pr[w]);
            }
          }
          if (BWD) {
            f32x4 gr;
#pragma unroll
            for (int w = 0; w < 4; ++w) gr[w] = d[w] * (pr[w] - float(lab[w] == c));
            store_stream<NT>(reinterpret_cast<f32x4 *>(ds + size_t(c) * P), gr);
          }
        }
      }
      if (NLL && phase == 0u) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          if (lab[w] >= C) nll[pix + uint32_t(w)] = ignore ? 0.0f : __builtin_nanf("");
        }
      }
    }
  }
}

// The tile a shape takes.  512 threads; 8 slots per thread up to 128 classes (256 on planes that are not whole
// 128-byte lines), 16 up to 512, 32 beyond (some 170 registers: one workgroup per CU, which still reads x once where
// the two-pass kernel reads it twice -- [1024, 1000] 3.0 -> 4.2 TB/s, [65536, 1000] 3.5 -> 4.4, [196, 800] 2.3 -> 3.7); runs of as many pixel groups as the threads then hold, up to 32 (64 up to 64 classes, 24
// on planes that are not whole lines: [900, 100] 5.6 TB/s in runs of 24 groups, 5.4 in runs of 32), a multiple of 8
// groups on planes of whole lines and of 4 otherwise, evened out over the tiles of a plane without adding a tile.
// (Shorter runs that divide the plane exactly were slower where they fell under 16 groups: [324, 100] in runs of 12
// 3.7 TB/s, of 24 5.5.)
// Measured alternatives: 256 and 1024 threads are within a few per cent either way at most shapes and 10 % behind at
// some; dealing the tiles per XCD costs 3-7 % on planes of whole lines.
ColReg nd_col_reg(uint32_t P, uint32_t C) {
  ColReg cr = {0, 0, 0, 0, 0, false};
  if (tuning().nd_colreg == 0) return cr;
  if (C <= 32u || C > 1024u) return cr;
  // Shorter planes keep the kernels tuned for them (whole samples in registers, the LDS tiles), except planes of 16
  // pixels and more that are not whole 16-byte groups from 129 classes on, which none of those takes well:
  // [49, 300] 1.6 -> 4.8 TB/s, [25, 512] 1.3 -> 5.3, [121, 150] 2.6 -> 5.1, [17, 200] 2.2 -> 5.4 (at 65 classes the
  // LDS tiles are faster, 4.0-4.9 against 2.1-4.0, at 100 it depends on the plane), and planes of whole groups from 513
  // classes on, which no form of the sample kernel holds: [16, 1000] 3.0 -> 5.3, [64, 944] 3.1 -> 4.5.
  if (P < 128u && ((P % 4u == 0 && C <= 512u) || P < 16u || C < 129u)) return cr;
  const uint32_t P4 = (P + 3u) / 4u;  // (planes that are not whole 16-byte groups: the last group ends with the plane)
  const bool lines = P % 32u == 0;
  const uint32_t ns = (C <= 128u || (!lines && C <= 256u)) ? 8u : (C <= 512u ? 16u : 32u);
  const uint32_t ph_need = (C + ns - 1u) / ns;  // at most 32
  const uint32_t step = lines ? 8u : 4u;
  uint32_t gt_max = 512u / ph_need;
  const uint32_t cap = C <= 64u ? 64u : (lines ? 32u : 24u);
  if (gt_max > cap) gt_max = cap;
  gt_max &= ~(step - 1u);
  if (gt_max < step) gt_max = step;  // (512 / 32 = 16 groups at the least: never below a step)
  // Planes of up to 1024 pixels where the plane and the sample are powers of two: runs one step shorter, which do not
  // divide the plane, so that the tiles of a plane are not all alike: [1024, 64] 5.0 TB/s in four runs of 64 groups per
  // 4 KB plane, 6.2 in runs of 56; [1024, 256] 5.4 -> 5.7 and [512, 256] 5.2 -> 5.6 in runs of 24 instead of 32,
  // [1024, 128] 5.8 -> 6.0.  (Longer planes prefer the even division: [2048, 256] 5.9 in runs of 32, 5.6 in runs of 24;
  // so do other class counts: [1024, 33 / 48 / 56] 6.2-6.3 in runs of 64, 5.7-5.8 in runs of 56.)
  const bool pow2_sample = P4 <= 256u && (P & (P - 1u)) == 0 && (C & (C - 1u)) == 0;
  if (pow2_sample && gt_max >= 3u * step && P4 > gt_max) gt_max -= step;  // (not below 16 groups)
  uint32_t Gt = P4;
  if (P4 > gt_max) {
    // as many tiles per plane as runs of gt_max groups make, evened out ([196, 300]: 49 groups as 20 + 20 + 9 instead
    // of 24 + 24 + 1)
    const uint32_t per_plane = (P4 + gt_max - 1u) / gt_max;
    Gt = ((P4 + per_plane - 1u) / per_plane + step - 1u) & ~(step - 1u);
  }
  uint32_t PH = 512u / Gt;
  if (PH > 32u) PH = 32u;
  if (uint64_t(PH) * ns < C) return cr;
  cr.ns = ns;
  cr.Gt = Gt;
  cr.PH = PH;
  cr.tiles = (P4 + Gt - 1u) / Gt;
  // (planes that are not whole lines: neighbouring tiles, which share lines, on one XCD -- [16385, 100] 3.8 -> 5.3 TB/s,
  // [4225, 150] 3.9 -> 4.9; one shape measured loses, [65535, 64] 4.8 -> 3.8)
  cr.xcd = lines ? 0u : 1u;
  cr.fits = true;
  return cr;
}

template <bool NLL, bool BWD>
void launch_softmax_nd_colreg(const ColReg &cr, uint32_t P, uint32_t C, uint32_t N, const float *x, float *y,
                              const uint32_t *cat, float *nll, const float *dy, float *dx, bool ignore,
                              hipStream_t s) {
  const uint64_t total = uint64_t(cr.tiles) * N;  // at most len / 128: a tile is 33 classes of 4 pixel groups or more
  uint32_t max_blocks = 1u << 24;
  if (tuning().flat_wg_per_cu > 0) max_blocks = uint32_t(device_cu_count()) * uint32_t(tuning().flat_wg_per_cu);  // (the tests' way into the loop over tiles)
  const uint32_t blocks = total < max_blocks ? uint32_t(total) : max_blocks;
  const uint32_t launch_threads = (cr.Gt * cr.PH + kWave - 1u) / kWave * kWave;
  const FastDiv div_gt(cr.Gt), div_tiles(cr.tiles);
  // streaming stores only where every run of a tile is whole 64-byte pieces
  const bool whole_pieces = P % 16u == 0 && cr.Gt % 4u == 0;
  const int nt = whole_pieces ? policy_for_outputs(stream_policy(size_t(P) * C * N * sizeof(float), tuning().nontemporal), y, dx) : 0;
  with_stream_policy(nt, [&](auto policy) {
    constexpr int NT = decltype(policy)::value;
    if (cr.ns == 8) {
      softmax_nd_colreg_kernel<8, 512, NLL, BWD, NT><<<blocks, launch_threads, 0, s>>>(
          P, C, cr.Gt, cr.PH, uint32_t(total), div_gt, div_tiles, ignore ? 1u : 0u, cr.xcd, x, y, cat, nll, dy, dx);
    } else if (cr.ns == 32) {
      softmax_nd_colreg_kernel<32, 512, NLL, BWD, NT><<<blocks, launch_threads, 0, s>>>(
          P, C, cr.Gt, cr.PH, uint32_t(total), div_gt, div_tiles, ignore ? 1u : 0u, cr.xcd, x, y, cat, nll, dy, dx);
    } else {
      softmax_nd_colreg_kernel<16, 512, NLL, BWD, NT><<<blocks, launch_threads, 0, s>>>(
          P, C, cr.Gt, cr.PH, uint32_t(total), div_gt, div_tiles, ignore ? 1u : 0u, cr.xcd, x, y, cat, nll, dy, dx);
    }
  });
}

// Which kernel takes 33 to 128 classes: one pixel per thread where 16-byte accesses are not legal, or where the
// planes are so short that eight lanes per pixel group would read 128-byte pieces of them (P = 196, C = 64:
// 3.7 TB/s against 2.3).  The plain and the fused entry points must agree on this: the order in which a pixel's
// exponentials are added, hence the bits of p, depends on the kernel.
bool nd_one_pixel_per_thread(uint32_t P, uint32_t C, bool vec) { return (!vec || P < 1024) && C > 32 && C <= 128; }

// whether the n-d entry points take their 16-byte kernels: planes of whole 16-byte groups; where the arrays lie
// does not matter (the accesses only ask for 4-byte alignment), so every entry point picks the same kernel family
// for a shape and a pixel's sum is added in the same order by all of them
bool nd_vec(uint32_t P) { return P % 4 == 0; }

// Planes that are not whole 16-byte groups, up to 32 classes: the two-lane kernel over groups of four pixels all the
// same, 16-byte accesses at 4-byte-aligned addresses, the last group of a plane moved back to end with the plane
// (PixelGrid).  Against one pixel per thread: [4225, 2] 4.5 -> 5.8 TB/s, [1025, 4] 4.9 -> 5.8, [4225, 19] 5.0 -> 5.2,
// [263169, 21] 4.3 -> 4.9 (what is left to the aligned rate, 6.0, is the stores that straddle 16-byte groups).
bool nd_overlapped_pairs(uint32_t P, uint32_t C) { return P % 4 != 0 && P >= 8 && C <= 32; }

// Which kernel family a shape takes: one decision for the plain and the fused entry points, because the order in
// which a pixel's exponentials are added, hence the bits of p, follows the kernel.  `separate` says that no output
// array is the input array: planes that are not whole 16-byte groups need that for their 16-byte kernels, whose last
// two groups of a plane overlap (with y == x such shapes take the kernels with one pixel per thread, whose sums are
// added in another order; nothing else depends on the arrays).
enum class NdFamily : uint32_t {
  Rows = 0,        // P == 1
  SampleReg = 1,   // whole samples in registers
  Tile = 2,        // whole samples through an LDS tile
  ColReg = 3,      // column tiles in registers
  ColTile = 4,     // column tiles in LDS
  PixelPerThread = 5,  // 33 to 128 classes, one pixel per thread (4-byte accesses)
  Groups16 = 6,    // groups of four pixels: two lanes per group up to 32 classes, eight up to 256, two passes beyond
  Singles = 7,     // single pixels: registers up to 32 classes, two passes beyond
};
struct NdPlan {
  NdFamily family;
  SampleReg sr;
  ColReg cr;
  ColTile ct;
};

NdPlan nd_plan(uint32_t P, uint32_t C, bool separate) {
  NdPlan pl = {NdFamily::Singles, {0, 0, 0, 0, false}, {0, 0, 0, 0, 0, false}, {0, 0, 0, false}};
  if (P == 1) {
    pl.family = NdFamily::Rows;
    return pl;
  }
  const bool vec = nd_vec(P);
  pl.sr = nd_sample_reg(P, C);
  if (pl.sr.fits) {
    pl.family = NdFamily::SampleReg;
    return pl;
  }
  if (nd_tile_fits(P, C)) {
    pl.family = NdFamily::Tile;
    return pl;
  }
  pl.cr = nd_col_reg(P, C);
  if (pl.cr.fits && (vec || separate)) {
    pl.family = NdFamily::ColReg;
    return pl;
  }
  pl.ct = nd_col_tile(P, C);
  if (vec && pl.ct.fits) {
    pl.family = NdFamily::ColTile;
    return pl;
  }
  if (nd_one_pixel_per_thread(P, C, vec)) {
    pl.family = NdFamily::PixelPerThread;
    return pl;
  }
  if (vec || (nd_overlapped_pairs(P, C) && separate)) pl.family = NdFamily::Groups16;
  return pl;
}

void launch_softmax_nd(const char *symbol, uint32_t P, uint32_t C, uint32_t N, const float *x, float *y,
                       CUstream_st *stream) {
  const uint32_t len = checked_len(P, C, N, symbol);
  if (len == 0) return;
  if (P == 1) {  // the class axis is contiguous: this is the row form
    launch_softmax_rows(symbol, C, N, x, y, stream);
    return;
  }
  hipStream_t s = as_stream(stream);
  const NdPlan pl = nd_plan(P, C, x != y);
  switch (pl.family) {
    case NdFamily::Rows:  // (taken above)
      break;
    case NdFamily::SampleReg:
      launch_softmax_nd_samplereg<false, false>(pl.sr, P, C, N, x, y, nullptr, nullptr, nullptr, nullptr, false, s);
      break;
    case NdFamily::Tile:
      launch_softmax_nd_tile<false, false>(P, C, N, x, y, nullptr, nullptr, nullptr, nullptr, false, s);
      break;
    case NdFamily::ColReg:
      launch_softmax_nd_colreg<false, false>(pl.cr, P, C, N, x, y, nullptr, nullptr, nullptr, nullptr, false, s);
      break;
    case NdFamily::ColTile:
      launch_softmax_nd_coltile<false, false>(pl.ct, P, C, N, x, y, nullptr, nullptr, nullptr, nullptr, false, s);
      break;
    case NdFamily::PixelPerThread: {
      // one pixel per thread keeps the row in registers and is still coalesced across the wave
      const PixelGrid pg = make_pixel_grid(P, C, N, 1);
      const uint32_t blocks = pixel_blocks(pg.total_groups);
      if (C <= 64) {
        softmax_nd_reg_kernel<64, float, false, 0, 1><<<blocks, kBlock, 0, s>>>(pg, x, y, nullptr, nullptr);
      } else {
        softmax_nd_reg_kernel<128, float, false, 0, 1><<<blocks, kBlock, 0, s>>>(pg, x, y, nullptr, nullptr);
      }
      break;
    }
    case NdFamily::Groups16:
      launch_softmax_nd_typed<f32x4>(P, C, N, x, y, s);
      break;
    case NdFamily::Singles:
      launch_softmax_nd_typed<float>(P, C, N, x, y, s);
      break;
  }
  note_launch(symbol);
}

template <bool ACC>
void launch_softmax_cat_nll_bwd(const char *symbol, uint32_t K, uint32_t R, const float *dy, const float *prob,
                                const uint32_t *cat, float *dx, CUstream_st *stream, bool ignore = false) {
  launch_chan_map<1, ACC>(symbol, K, R, 1, CatNllBwdMap{dy, cat, K, ignore}, prob, nullptr, dx, stream);
}

void launch_softmax_cat_nll(const char *symbol, uint32_t K, uint32_t R, const float *prob, const uint32_t *cat,
                            float *nll, CUstream_st *stream, bool ignore) {
  (void)checked_len(K, R, 1, symbol);
  if (R == 0) return;
  softmax_cat_nll_kernel<<<stream_grid(R, 1), kBlock, 0, as_stream(stream)>>>(K, R, prob, cat, nll, ignore);
  note_launch(symbol);
}

void launch_softmax_nd_cat_nll(const char *symbol, uint32_t P, uint32_t C, uint32_t N, const float *prob,
                               const uint32_t *cat, float *nll, CUstream_st *stream, bool ignore) {
  (void)checked_len(P, C, N, symbol);
  if (P == 0 || N == 0) return;
  if (P % 4 == 0) {
    PixelGrid pg = make_pixel_grid(P, C, N, 4, ignore);
    pg.xcd = (tuning().nd_xcd_mask & 4) ? 1u : 0u;
    softmax_nd_cat_nll_kernel<f32x4><<<pixel_blocks(pg.total_groups), kBlock, 0, as_stream(stream)>>>(pg, prob, cat, nll);
  } else {
    const PixelGrid pg = make_pixel_grid(P, C, N, 1, ignore);
    softmax_nd_cat_nll_kernel<float><<<pixel_blocks(pg.total_groups), kBlock, 0, as_stream(stream)>>>(pg, prob, cat, nll);
  }
  note_launch(symbol);
}

// The same map walked as the flat array it is: a thread takes one 16-byte group of dx (four consecutive pixels of
// one class), so a wave's accesses are 1 KiB contiguous however short the planes are, and fetches its pixels' dy and
// labels from the caches (every class of a sample asks for the same ones).  Taken for planes of up to
// nd_bwd_flat_max_plane pixels (131072: a sample's dy and labels, 8 bytes per pixel, then stay in the L2s while its
// classes go by): [196, 19, 18020] 3.6 -> 5.6 TB/s, [2048, 64, 512] 4.6 -> 5.8, [65536, 100, 10] 4.9 -> 5.8,
// accumulating 5.0 -> 6.3; at [524288, 19, 8] inside a softmax -> NLL -> backward sequence it loses to the kernel
// above, 127 us against 110.  The arithmetic is that of the kernel above.
template <bool ACC, int NT>
__global__ __launch_bounds__(kBlock) void softmax_nd_cat_nll_bwd_flat_kernel(uint32_t P, uint32_t C, uint32_t total_groups,
                                                                             FastDiv div_gpp, FastDiv div_c, uint32_t ignore,
                                                                             const float *__restrict__ dy,
                                                                             const float *__restrict__ prob,
                                                                             const uint32_t *__restrict__ cat,
                                                                             float *dx) {
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;  // 64-bit: index + stride can pass 2^32
  for (uint64_t g64 = uint64_t(blockIdx.x) * kBlock + threadIdx.x; g64 < total_groups; g64 += stride) {
    const uint32_t g = uint32_t(g64);
    uint32_t plane, r;  // plane = n * C + k, r = the group's place in the plane
    div_gpp.divmod(g, plane, r);
    const uint32_t n = div_c.div(plane);
    const uint32_t k = plane - n * C;
    const size_t pix = size_t(n) * P + size_t(r) * 4u;
    f32x4 d = load_stream<0>(reinterpret_cast<const f32x4 *>(dy + pix));
    const u32x4 lab = load_stream<0>(reinterpret_cast<const u32x4 *>(cat + pix));
    const f32x4 pr = load_stream<NT>(reinterpret_cast<const f32x4 *>(prob) + g);
    f32x4 old = {0.0f, 0.0f, 0.0f, 0.0f};
    if (ACC) old = load_stream<NT>(reinterpret_cast<const f32x4 *>(dx) + g);
    f32x4 out;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if (ignore && lab[w] >= C) d[w] = 0.0f;
      const float t = pr[w] - float(lab[w] == k);
      out[w] = ACC ? fmaf(d[w], t, old[w]) : d[w] * t;
    }
    store_stream<NT>(reinterpret_cast<f32x4 *>(dx) + g, out);
  }
}

// The flat walk for planes that are not whole 16-byte groups: a thread still takes one 16-byte group of dx, which now
// may lie across the end of a plane (its pixels then belong to two classes, or to two samples) or across the end of
// the array.  A group inside one plane fetches dy and labels with 16-byte accesses at 4-byte-aligned addresses; the
// one group per plane that lies across its end, and the array's last group, go element by element.  The stores stay
// aligned 16-byte ones, which the kernels with one pixel per thread do not have: [4225, 19] 4.3 -> 5.0 TB/s,
// [1025, 100] 3.2 -> 5.1, [961, 64] 4.0 -> 5.2, [65535, 4] 4.2 -> 5.1.
template <bool ACC, int NT>
__global__ __launch_bounds__(kBlock) void softmax_nd_cat_nll_bwd_flat_any_kernel(uint32_t P, uint32_t C, uint32_t len,
                                                                                 FastDiv div_p, FastDiv div_c,
                                                                                 uint32_t ignore,
                                                                                 const float *__restrict__ dy,
                                                                                 const float *__restrict__ prob,
                                                                                 const uint32_t *__restrict__ cat,
                                                                                 float *dx) {
  const uint64_t stride = uint64_t(gridDim.x) * kBlock;  // 64-bit: index + stride can pass 2^32
  const uint64_t total_groups = (uint64_t(len) + 3u) / 4u;  // (64-bit: len + 3 can pass 2^32)
  for (uint64_t g64 = uint64_t(blockIdx.x) * kBlock + threadIdx.x; g64 < total_groups; g64 += stride) {
    const uint32_t e = uint32_t(g64) * 4u;  // the group's first element: below len
    uint32_t plane, r;                      // plane = n * C + k, r = the pixel
    div_p.divmod(e, plane, r);
    if (r + 4u <= P && uint64_t(e) + 4u <= len) {
      const uint32_t n = div_c.div(plane);
      const uint32_t k = plane - n * C;
      const size_t pix = size_t(n) * P + r;
      f32x4 d = load_stream<0>(reinterpret_cast<const f32x4 *>(dy + pix));
      const u32x4 lab = load_stream<0>(reinterpret_cast<const u32x4 *>(cat + pix));
      const f32x4 pr = load_stream<NT>(reinterpret_cast<const f32x4 *>(prob + e));
      f32x4 old = {0.0f, 0.0f, 0.0f, 0.0f};
      if (ACC) old = load_stream<NT>(reinterpret_cast<const f32x4 *>(dx + e));
      f32x4 out;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        if (ignore && lab[w] >= C) d[w] = 0.0f;
        const float t = pr[w] - float(lab[w] == k);
        out[w] = ACC ? fmaf(d[w], t, old[w]) : d[w] * t;
      }
      store_stream<NT>(reinterpret_cast<f32x4 *>(dx + e), out);
    } else {
      // The group lies across the end of a plane (P >= 16: of one plane only) or of the array.  Its elements' planes
      // and pixels follow from the first one's; everything is requested before anything is used.
      uint32_t kk[4], label[4];
      size_t pix[4];
      float d[4], pr[4], old[4];
      bool in[4];
      const uint32_t n0 = div_c.div(plane);
      const uint32_t k0 = plane - n0 * C;
#pragma unroll
      for (uint32_t w = 0; w < 4u; ++w) {
        in[w] = uint64_t(e) + w < len;
        const bool next = r + w >= P;            // the element belongs to the next plane
        const uint32_t rr = next ? r + w - P : r + w;
        uint32_t k = next ? k0 + 1u : k0, n = n0;
        if (k == C) {                            // ... which is the first plane of the next sample
          k = 0u;
          n += 1u;
        }
        kk[w] = k;
        pix[w] = size_t(n) * P + rr;
      }
#pragma unroll
      for (uint32_t w = 0; w < 4u; ++w) {
        label[w] = in[w] ? cat[pix[w]] : 0u;
        d[w] = in[w] ? dy[pix[w]] : 0.0f;
        pr[w] = in[w] ? prob[e + w] : 0.0f;
        old[w] = (ACC && in[w]) ? dx[e + w] : 0.0f;
      }
#pragma unroll
      for (uint32_t w = 0; w < 4u; ++w) {
        if (ignore && label[w] >= C) d[w] = 0.0f;
        const float t = pr[w] - float(label[w] == kk[w]);
        if (in[w]) dx[e + w] = ACC ? fmaf(d[w], t, old[w]) : d[w] * t;
      }
    }
  }
}

// The backward pass is a map, so with few pixels and many classes the classes are shared out as well: runs of
// `chunk` classes (a multiple of 16: a thread reads its pixels' dy and labels once per run) over blockIdx.y, as
// many as it takes to give the GPU eight workgroups per CU ([65536, 256, 4]: 256 workgroups of pixel groups).
dim3 nd_bwd_grid(uint32_t total_groups, uint32_t C, uint32_t &chunk) {
  const uint32_t bx = pixel_blocks(total_groups);
  const uint32_t want = uint32_t(device_cu_count()) * 8u;
  uint32_t runs = bx >= want ? 1u : (want + bx - 1u) / bx;
  const uint32_t most = (C + 15u) / 16u;
  if (runs > most) runs = most;
  chunk = ((C + runs - 1u) / runs + 15u) / 16u * 16u;
  runs = (C + chunk - 1u) / chunk;
  return dim3(bx, runs, 1);
}

template <bool ACC>
void launch_softmax_nd_cat_nll_bwd(const char *symbol, uint32_t P, uint32_t C, uint32_t N, const float *dy,
                                   const float *prob, const uint32_t *cat, float *dx, CUstream_st *stream,
                                   bool ignore = false) {
  const uint32_t len = checked_len(P, C, N, symbol);
  if (len == 0) return;
  if (P == 1) {
    launch_softmax_cat_nll_bwd<ACC>(symbol, C, N, dy, prob, cat, dx, stream, ignore);
    return;
  }
  hipStream_t s = as_stream(stream);
  const bool vec = (P % 4 == 0);  // planes of whole 16-byte groups, wherever the arrays lie
  uint32_t chunk = C;
  if (vec && P <= uint32_t(tuning().nd_bwd_flat_max_plane)) {
    const uint32_t total_groups = len / 4u;
    const FastDiv div_gpp(P / 4u), div_c(C);
    with_stream_policy(policy_for_outputs(stream_policy(size_t(len) * sizeof(float), tuning().nontemporal), dx), [&](auto policy) {
      softmax_nd_cat_nll_bwd_flat_kernel<ACC, decltype(policy)::value>
          <<<stream_grid(total_groups, 1), kBlock, 0, s>>>(P, C, total_groups, div_gpp, div_c, ignore ? 1u : 0u, dy, prob,
                                                          cat, dx);
    });
  } else if (!vec && P >= (ACC ? 200u : 64u) && P <= uint32_t(tuning().nd_bwd_flat_max_plane)) {
    // (shorter planes: every wave of 256 elements then holds groups that lie across the end of a plane and go
    // element by element.  One pixel per thread is faster below 64 pixels, [33, 19] 3.8 TB/s against 2.7, and when
    // accumulating below some 200, [129, 19] 4.7 against 4.3; above, [361, 19] 4.0 -> 4.7 and accumulating 4.7 -> 5.0,
    // [129, 100] 3.1 -> 4.7.)
    const FastDiv div_p(P), div_c(C);
    with_stream_policy(policy_for_outputs(stream_policy(size_t(len) * sizeof(float), tuning().nontemporal), dx), [&](auto policy) {
      softmax_nd_cat_nll_bwd_flat_any_kernel<ACC, decltype(policy)::value>
          <<<stream_grid((uint64_t(len) + 3u) / 4u, 1), kBlock, 0, s>>>(P, C, len, div_p, div_c, ignore ? 1u : 0u, dy, prob,
                                                                       cat, dx);
    });
  } else if (vec) {
    PixelGrid pg = make_pixel_grid(P, C, N, 4, ignore);
    pg.xcd = (tuning().nd_xcd_mask & 2) ? 1u : 0u;
    const dim3 grid = nd_bwd_grid(pg.total_groups, C, chunk);
    const int nt = (P % 16u == 0) ? policy_for_outputs(stream_policy(size_t(len) * sizeof(float), tuning().nontemporal), dx) : 0;
    with_stream_policy(nt, [&](auto policy) {
      softmax_nd_cat_nll_bwd_kernel<f32x4, ACC, decltype(policy)::value>
          <<<grid, kBlock, 0, s>>>(pg, dy, prob, cat, dx, chunk);
    });
  } else {
    const PixelGrid pg = make_pixel_grid(P, C, N, 1, ignore);
    const dim3 grid = nd_bwd_grid(pg.total_groups, C, chunk);
    softmax_nd_cat_nll_bwd_kernel<float, ACC, 0><<<grid, kBlock, 0, s>>>(pg, dy, prob, cat, dx, chunk);
  }
  note_launch(symbol);
}

}  // namespace
}  // namespace anode

using namespace anode;

ANODE_EXPORT void anode_gpu_softmax_packed_block_f32(uint32_t dim0, uint32_t dim1, const float *x, float *y,
                                                     const KernelConfig *, CUstream_st *stream) {
  launch_softmax_rows(__func__, dim0, dim1, x, y, stream);
}

ANODE_EXPORT void anode_gpu_softmax_packed_deterministic_f32(uint32_t dim0, uint32_t dim1, const float *x,
                                                             float *y, const KernelConfig *,
                                                             CUstream_st *stream) {
  launch_softmax_rows(__func__, dim0, dim1, x, y, stream);
}

ANODE_EXPORT void anode_gpu_softmax_cat_nll_packed_f32(uint32_t dim0, uint32_t dim1, const float *softmax,
                                                       const uint32_t *cat_data, float *nll,
                                                       const KernelConfig *, CUstream_st *stream) {
  launch_softmax_cat_nll(__func__, dim0, dim1, softmax, cat_data, nll, stream, false);
}

ANODE_EXPORT void anode_gpu_softmax_cat_nll_bwd_packed_f32(uint32_t dim0, uint32_t dim1, const float *dy,
                                                           const float *softmax, const uint32_t *cat_data,
                                                           float *dx, const KernelConfig *, CUstream_st *stream) {
  launch_softmax_cat_nll_bwd<false>(__func__, dim0, dim1, dy, softmax, cat_data, dx, stream);
}

ANODE_EXPORT void anode_gpu_softmax_cat_nll_bwd_packed_accumulate_f32(uint32_t dim0, uint32_t dim1,
                                                                      const float *dy, const float *softmax,
                                                                      const uint32_t *cat_data, float *dx,
                                                                      const KernelConfig *, CUstream_st *stream) {
  launch_softmax_cat_nll_bwd<true>(__func__, dim0, dim1, dy, softmax, cat_data, dx, stream);
}

ANODE_EXPORT void anode_gpu_softmax_nd_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1,
                                                  const float *x, float *y, const KernelConfig *,
                                                  CUstream_st *stream) {
  launch_softmax_nd(__func__, prefix_dim, dim0, dim1, x, y, stream);
}

ANODE_EXPORT void anode_gpu_softmax_nd_cat_nll_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1,
                                                          const float *softmax, const uint32_t *cat_data,
                                                          float *nll, const KernelConfig *, CUstream_st *stream) {
  launch_softmax_nd_cat_nll(__func__, prefix_dim, dim0, dim1, softmax, cat_data, nll, stream, false);
}

ANODE_EXPORT void anode_gpu_softmax_nd_cat_nll_bwd_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1,
                                                              const float *dy, const float *softmax,
                                                              const uint32_t *cat_data, float *dx,
                                                              const KernelConfig *, CUstream_st *stream) {
  launch_softmax_nd_cat_nll_bwd<false>(__func__, prefix_dim, dim0, dim1, dy, softmax, cat_data, dx, stream);
}

ANODE_EXPORT void anode_gpu_softmax_nd_cat_nll_bwd_packed_accumulate_f32(uint32_t prefix_dim, uint32_t dim0,
                                                                         uint32_t dim1, const float *dy,
                                                                         const float *softmax,
                                                                         const uint32_t *cat_data, float *dx,
                                                                         const KernelConfig *,
                                                                         CUstream_st *stream) {
  launch_softmax_nd_cat_nll_bwd<true>(__func__, prefix_dim, dim0, dim1, dy, softmax, cat_data, dx, stream);
}

// Additive (no counterpart in the reference): row softmax and softmax_cat_nll in one pass over x (the recipe of
// src/ops.rs:1172-1176 as one launch).  Writes the same probabilities and the same nll values as the two entry
// points: the thread that stores the label's probability also writes -log of it.
ANODE_EXPORT void anode_gpu_softmax_cat_nll_fused_packed_f32(uint32_t dim0, uint32_t dim1, const float *x,
                                                             const uint32_t *cat_data, float *softmax, float *nll,
                                                             const KernelConfig *, CUstream_st *stream) {
  launch_softmax_rows(__func__, dim0, dim1, x, softmax, stream, RowNll{cat_data, nll, false, nullptr, nullptr});
}

// Additive: the same with the backward of the NLL as well, for callers that know the upstream gradient dy before the
// forward pass (a summed or averaged loss): dx = dy * (softmax - onehot), the values of
// anode_gpu_softmax_cat_nll_bwd_packed_f32, from the same launch.  A [256,1000] head is launch-bound: one launch
// instead of three.
ANODE_EXPORT void anode_gpu_softmax_cat_nll_fused_fwd_bwd_packed_f32(uint32_t dim0, uint32_t dim1, const float *x,
                                                                     const uint32_t *cat_data, const float *dy,
                                                                     float *softmax, float *nll, float *dx,
                                                                     const KernelConfig *, CUstream_st *stream) {
  launch_softmax_rows(__func__, dim0, dim1, x, softmax, stream, RowNll{cat_data, nll, false, dy, dx});
}

// The fused n-d entry points: the kernel that nd_plan() names for the shape, with the label gather (and the backward
// pass) riding along; shapes whose kernel has no such form run the separate launches back to back.
template <bool BWD>
static void launch_softmax_nd_fused(const char *symbol, uint32_t P, uint32_t C, uint32_t N, const float *x,
                                    const uint32_t *cat, const float *dy, float *softmax, float *nll, float *dx,
                                    const KernelConfig *cfg, CUstream_st *stream) {
  const uint32_t len = checked_len(P, C, N, symbol);
  if (len == 0) return;
  hipStream_t s = as_stream(stream);
  const NdPlan pl = nd_plan(P, C, x != softmax && (!BWD || x != dx));
  bool launched = true;
  switch (pl.family) {
    case NdFamily::Rows:  // the class axis is contiguous: the row form
      launch_softmax_rows(symbol, C, N, x, softmax, stream, RowNll{cat, nll, false, BWD ? dy : nullptr, BWD ? dx : nullptr});
      return;
    case NdFamily::SampleReg:
      launch_softmax_nd_samplereg<true, BWD>(pl.sr, P, C, N, x, softmax, cat, nll, dy, dx, false, s);
      break;
    case NdFamily::Tile:
      launch_softmax_nd_tile<true, BWD>(P, C, N, x, softmax, cat, nll, dy, dx, false, s);
      break;
    case NdFamily::ColReg:
      launch_softmax_nd_colreg<true, BWD>(pl.cr, P, C, N, x, softmax, cat, nll, dy, dx, false, s);
      break;
    case NdFamily::ColTile:
      launch_softmax_nd_coltile<true, BWD>(pl.ct, P, C, N, x, softmax, cat, nll, dy, dx, false, s);
      break;
    case NdFamily::Groups16:
      if (C <= 256) {
        launch_softmax_nd_reg<f32x4, true, BWD>(P, C, N, x, softmax, cat, nll, s, dy, dx);
      } else {
        launched = false;
      }
      break;
    case NdFamily::Singles:
      if (C <= 32) {
        launch_softmax_nd_reg<float, true, BWD>(P, C, N, x, softmax, cat, nll, s, dy, dx);
      } else {
        launched = false;
      }
      break;
    case NdFamily::PixelPerThread:
      launched = false;
      break;
  }
  if (launched) {
    note_launch(symbol);
    return;
  }
  // shapes outside the kernels that carry the labels along: the separate passes, back to back
  anode_gpu_softmax_nd_packed_f32(P, C, N, x, softmax, cfg, stream);
  anode_gpu_softmax_nd_cat_nll_packed_f32(P, C, N, softmax, cat, nll, cfg, stream);
  if (BWD) anode_gpu_softmax_nd_cat_nll_bwd_packed_f32(P, C, N, dy, softmax, cat, dx, cfg, stream);
}

// Additive (no counterpart in the reference): softmax_nd and softmax_nd_cat_nll in one pass over x.
// Writes the same probabilities and the same nll values as the two separate entry points.
ANODE_EXPORT void anode_gpu_softmax_nd_cat_nll_fused_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1,
                                                                const float *x, const uint32_t *cat_data,
                                                                float *softmax, float *nll, const KernelConfig *cfg,
                                                                CUstream_st *stream) {
  launch_softmax_nd_fused<false>(__func__, prefix_dim, dim0, dim1, x, cat_data, nullptr, softmax, nll, nullptr, cfg, stream);
}

// Additive: the same and the backward pass for a dy that is known before the forward pass (ones for a summed loss,
// 1/count for a mean), one launch instead of three.  softmax, nll and dx are bit-identical to softmax_nd,
// softmax_nd_cat_nll and softmax_nd_cat_nll_bwd.
ANODE_EXPORT void anode_gpu_softmax_nd_cat_nll_fused_fwd_bwd_packed_f32(uint32_t prefix_dim, uint32_t dim0,
                                                                        uint32_t dim1, const float *x,
                                                                        const uint32_t *cat_data, const float *dy,
                                                                        float *softmax, float *nll, float *dx,
                                                                        const KernelConfig *cfg, CUstream_st *stream) {
  launch_softmax_nd_fused<true>(__func__, prefix_dim, dim0, dim1, x, cat_data, dy, softmax, nll, dx, cfg, stream);
}

// Host-only view of nd_plan() for the tests: family, then the tiling of the family as 7 words (SampleReg: threads,
// slots, G, PH; ColReg: 512, slots, Gt, PH, tiles per plane, xcd; ColTile: TP, L, tiles per plane).
ANODE_EXPORT void anode_gpu_softmax_nd_plan_probe(uint32_t P, uint32_t C, int separate, uint32_t *out8) {
  const NdPlan pl = nd_plan(P, C, separate != 0);
  uint32_t v[8] = {uint32_t(pl.family), 0, 0, 0, 0, 0, 0, 0};
  if (pl.family == NdFamily::SampleReg) {
    v[1] = pl.sr.threads; v[2] = pl.sr.ns; v[3] = pl.sr.G; v[4] = pl.sr.PH;
  } else if (pl.family == NdFamily::ColReg) {
    v[1] = 512; v[2] = pl.cr.ns; v[3] = pl.cr.Gt; v[4] = pl.cr.PH; v[5] = pl.cr.tiles; v[6] = pl.cr.xcd;
  } else if (pl.family == NdFamily::ColTile) {
    v[1] = pl.ct.TP; v[2] = pl.ct.L; v[3] = pl.ct.tiles_per_sample;
  }
  std::memcpy(out8, v, sizeof(v));
}

// Additive "ignore" variants (no counterpart in the reference, whose kernels give NaN and an unmasked gradient for
// a label >= the number of classes, softmax.cu:294-296, :331): such a row or pixel contributes nll = 0 and dx = 0
// (for _accumulate: dx unchanged).  In-range labels give bit-identical results to the plain entry points.
ANODE_EXPORT void anode_gpu_softmax_cat_nll_ignore_packed_f32(uint32_t dim0, uint32_t dim1, const float *softmax,
                                                              const uint32_t *cat_data, float *nll,
                                                              const KernelConfig *, CUstream_st *stream) {
  launch_softmax_cat_nll(__func__, dim0, dim1, softmax, cat_data, nll, stream, true);
}

ANODE_EXPORT void anode_gpu_softmax_cat_nll_bwd_ignore_packed_f32(uint32_t dim0, uint32_t dim1, const float *dy,
                                                                  const float *softmax, const uint32_t *cat_data,
                                                                  float *dx, const KernelConfig *,
                                                                  CUstream_st *stream) {
  launch_softmax_cat_nll_bwd<false>(__func__, dim0, dim1, dy, softmax, cat_data, dx, stream, true);
}

ANODE_EXPORT void anode_gpu_softmax_cat_nll_bwd_ignore_packed_accumulate_f32(uint32_t dim0, uint32_t dim1,
                                                                             const float *dy, const float *softmax,
                                                                             const uint32_t *cat_data, float *dx,
                                                                             const KernelConfig *,
                                                                             CUstream_st *stream) {
  launch_softmax_cat_nll_bwd<true>(__func__, dim0, dim1, dy, softmax, cat_data, dx, stream, true);
}

ANODE_EXPORT void anode_gpu_softmax_nd_cat_nll_ignore_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1,
                                                                 const float *softmax, const uint32_t *cat_data,
                                                                 float *nll, const KernelConfig *,
                                                                 CUstream_st *stream) {
  launch_softmax_nd_cat_nll(__func__, prefix_dim, dim0, dim1, softmax, cat_data, nll, stream, true);
}

ANODE_EXPORT void anode_gpu_softmax_nd_cat_nll_bwd_ignore_packed_f32(uint32_t prefix_dim, uint32_t dim0,
                                                                     uint32_t dim1, const float *dy,
                                                                     const float *softmax, const uint32_t *cat_data,
                                                                     float *dx, const KernelConfig *,
                                                                     CUstream_st *stream) {
  launch_softmax_nd_cat_nll_bwd<false>(__func__, prefix_dim, dim0, dim1, dy, softmax, cat_data, dx, stream, true);
}

ANODE_EXPORT void anode_gpu_softmax_nd_cat_nll_bwd_ignore_packed_accumulate_f32(uint32_t prefix_dim, uint32_t dim0,
                                                                                uint32_t dim1, const float *dy,
                                                                                const float *softmax,
                                                                                const uint32_t *cat_data, float *dx,
                                                                                const KernelConfig *,
                                                                                CUstream_st *stream) {
  launch_softmax_nd_cat_nll_bwd<true>(__func__, prefix_dim, dim0, dim1, dy, softmax, cat_data, dx, stream, true);
}
