// Per-channel reductions over a packed [S, C, N] array (S fastest):
//   out[c] = finalize(c, sum_{s,n} term0(a, b), sum_{s,n} term1(a, b)).
//
// One channel of a batch is N separate runs of S contiguous floats, and the
// number of channels is often far smaller than the number of compute units, so
// the work is cut into tiles that are independent of C:
//
//   "chunk" tiles (S large): SB contiguous positions of one (n, c) run, for NB
//     consecutive samples.  Every element of the tile belongs to one channel;
//     threads stream 16-byte groups and keep a few fp64 running sums.
//   "whole" tiles (S <= 4096): CB whole channels that are adjacent in memory
//     (CB*S contiguous floats), for NB consecutive samples.  A thread owns
//     fixed positions of that span and adds the same positions of every sample
//     into per-position fp64 sums, so accesses stay contiguous and 16-byte wide
//     even when S is odd; at the end of the tile the positions are folded to
//     channels through LDS.
//
// Each tile leaves one fp64 partial per (channel, tile) in a scratch buffer
// and a second, tiny kernel adds a channel's partials in a fixed order and
// applies the operator's finalisation.  All sums are fp64 and every order of
// addition is fixed by the launch geometry, so results are reproducible from
// run to run and independent of scheduling.  When a channel has a single
// partial the first kernel finalises directly.
#pragma once

#include "chan_map.hpp"
#include "common.hpp"

namespace anode {

// Positions of a "whole" tile: 1024, 2048 or 4096 (8 to 32 KiB of fp64 in LDS), the smallest that holds the tile.
// A narrow tile over more samples reads the same bytes as a wide one over fewer, but its epilogue (per-position sums
// through LDS) is a quarter of the work, it leaves room for four times as many workgroups per compute unit and a
// thread carries 4 instead of 16 running sums per statistic.
constexpr uint32_t kTilePos = 4096;     // the widest tile: bounds S of the whole-channel form
constexpr uint32_t kTilePosMin = 1024;  // the narrowest: one 16-byte group per thread
// LDS slot of tile position p in a tile of P positions.  A thread owns four consecutive positions; storing them in
// four planes lets the 64 lanes of a wave write consecutive doubles, and the plane pitch (P/4 + 16 doubles, i.e. 32
// banks off a multiple of 64) keeps the channel-wise read of consecutive positions at two lanes per bank pair, the
// minimum for 8-byte accesses.  (Stored in position order, every eighth lane hit the same banks: 45 % of the LDS
// cycles were conflicts.)
template <uint32_t P>
__host__ __device__ inline uint32_t tile_slot(uint32_t p) { return (p & 3u) * (P / 4 + 16) + (p >> 2); }
constexpr uint32_t kMaxTileChans = 256;

struct ReducePlan {
  uint32_t S, C, N;
  uint32_t whole;     // 0: chunk tiles, 1: wide whole-channel tiles, 2: lane tiles
  uint32_t CB;        // channels per tile (whole)
  uint32_t SB;        // positions per tile (chunk)
  uint32_t n_ctiles;  // whole: ceil(C / CB); chunk: C
  uint32_t n_stiles;  // whole: 1; chunk: ceil(S / SB)
  uint32_t NB;        // samples per tile
  uint32_t n_ntiles;  // ceil(N / NB)
  uint32_t ppc;       // partials per channel = n_stiles * n_ntiles
  uint32_t vec;       // 1: 16-byte accesses are legal for this geometry
  uint32_t grid;      // n_ctiles * n_stiles * n_ntiles
  uint32_t P;         // wide tiles: positions per tile (1024, 2048 or 4096); otherwise 0
  uint32_t J;         // lane tiles: samples that the lanes of a workgroup take side by side; otherwise 0
};

// Host-side tiling decision; `ptrs_aligned` says whether the 16-byte tilings
// may be taken (the launcher always says yes: loads only need 4-byte alignment;
// the 4-byte tilings remain for the geometries that have no 16-byte form and
// for the planner's tests), `nin` how many element arrays the reduction reads.  Exposed (anode_gpu_plan_reduce) so that it can be
// checked without a device.
ReducePlan plan_chan_reduce(uint32_t S, uint32_t C, uint32_t N, bool ptrs_aligned, uint32_t wg_target, int nin);

#if defined(__HIPCC__)

// Op concept:
//   static constexpr int NIN  (1 to 3 element inputs), NACC (1 to 3 sums);
//   struct Param;  __device__ Param load(uint32_t c) const;
//   __device__ void term(const Param&, float a, float b, double &s0, double &s1, double &s2) const;
//     (NIN == 3: term3(const Param&, float a, float b, float c, double &s0, double &s1, double &s2))
//   __device__ void finalize(uint32_t c, double s0, double s1, double s2) const;   // writes the output(s)

template <typename Op, typename P>
__device__ inline void chan_reduce_term(const Op &op, const P &prm, float a, float b, float c, double &s0,
                                        double &s1, double &s2) {
  if constexpr (Op::NIN >= 3) {
    op.term3(prm, a, b, c, s0, s1, s2);
  } else {
    op.term(prm, a, b, s0, s1, s2);
  }
}

template <typename Op, typename V, int NT>
__global__ __launch_bounds__(kBlock) void chan_reduce_chunk_kernel(ReducePlan pl, Op op,
                                                                   const float *__restrict__ a,
                                                                   const float *__restrict__ b,
                                                                   const float *__restrict__ c3,
                                                                   double *__restrict__ part) {
  constexpr int W = VecLanes<V>::n;
  constexpr int U = 4;
  __shared__ double lds[kBlock / kWave];

  const uint32_t st = blockIdx.x % pl.n_stiles;
  const uint32_t r = blockIdx.x / pl.n_stiles;
  const uint32_t c = r % pl.C;
  const uint32_t nt = r / pl.C;
  const uint32_t s0 = st * pl.SB;
  const uint32_t sl = min(pl.SB, pl.S - s0);
  const uint32_t LG = sl / uint32_t(W);
  const uint32_t n0 = nt * pl.NB;
  const uint32_t n1 = min(pl.N, n0 + pl.NB);
  const typename Op::Param prm = op.load(c);

  double acc0[U], acc1[U], acc2[U];
#pragma unroll
  for (int u = 0; u < U; ++u) acc0[u] = acc1[u] = acc2[u] = 0.0;

  for (uint32_t n = n0; n < n1; ++n) {
    const size_t row = (size_t(n) * pl.C + c) * pl.S + s0;
    const V *pa = reinterpret_cast<const V *>(a + row);
    const V *pb = reinterpret_cast<const V *>(b + row);
    const V *pc = reinterpret_cast<const V *>(c3 + row);
    for (uint32_t jb = 0; jb < LG; jb += uint32_t(U) * kBlock) {
      V va[U], vb[U], vc[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        // Every slot is loaded, a slot past the tile's end from the tile's last group again (and left out of the
        // sums below): with a branch round each load the compiler waits for the previous load before it issues
        // the next one.  (LG >= 1: a tile is never empty.)
        const uint32_t j = jb + uint32_t(u) * kBlock + threadIdx.x;
        const uint32_t jc = j < LG ? j : LG - 1u;
        va[u] = load_stream<NT>(&pa[jc]);
        if (Op::NIN >= 2) vb[u] = load_stream<NT>(&pb[jc]);
        if (Op::NIN >= 3) vc[u] = load_stream<NT>(&pc[jc]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t j = jb + uint32_t(u) * kBlock + threadIdx.x;
        if (j < LG) {
#pragma unroll
          for (int k = 0; k < W; ++k) {
            chan_reduce_term(op, prm, lane_get<V>(va[u], k), (Op::NIN >= 2) ? lane_get<V>(vb[u], k) : 0.0f,
                             (Op::NIN >= 3) ? lane_get<V>(vc[u], k) : 0.0f, acc0[u], acc1[u], acc2[u]);
          }
        }
      }
    }
  }

  double t0 = (acc0[0] + acc0[1]) + (acc0[2] + acc0[3]);
  double t1 = (acc1[0] + acc1[1]) + (acc1[2] + acc1[3]);
  double t2 = (acc2[0] + acc2[1]) + (acc2[2] + acc2[3]);
  t0 = block_sum(t0, lds);
  if (Op::NACC >= 2) t1 = block_sum(t1, lds);
  if (Op::NACC >= 3) t2 = block_sum(t2, lds);
  if (threadIdx.x == 0) {
    if (pl.ppc == 1) {
      op.finalize(c, t0, t1, t2);
    } else {
      const size_t plane = size_t(pl.C) * pl.ppc;
      const size_t slot = size_t(c) * pl.ppc + (nt * pl.n_stiles + st);
      part[slot] = t0;
      if (Op::NACC >= 2) part[plane + slot] = t1;
      if (Op::NACC >= 3) part[2 * plane + slot] = t2;
    }
  }
}

template <typename Op, typename V, int NT, uint32_t P>
__global__ __launch_bounds__(kBlock) void chan_reduce_whole_kernel(ReducePlan pl, FastDiv div_s, Op op,
                                                                   const float *__restrict__ a,
                                                                   const float *__restrict__ b,
                                                                   const float *__restrict__ c3,
                                                                   double *__restrict__ part) {
  constexpr int W = VecLanes<V>::n;
  constexpr int G = int(P / kBlock) / W;  // position groups owned by a thread
  // samples loaded before any is consumed: about eight 16-byte (or thirty-two 4-byte) loads in flight per thread
  constexpr int LOADS = G * Op::NIN;
  constexpr int TARGET = (W == 1) ? 32 : 8;
  constexpr int STAGES = LOADS >= TARGET ? 1 : TARGET / LOADS;
  __shared__ double lds[P + 64];

  const uint32_t nt = blockIdx.x / pl.n_ctiles;
  const uint32_t ct = xcd_contiguous(blockIdx.x % pl.n_ctiles, pl.n_ctiles);
  const uint32_t c0 = ct * pl.CB;
  const uint32_t cb = min(pl.CB, pl.C - c0);
  const uint32_t LG = (cb * pl.S) / uint32_t(W);
  const uint32_t n0 = nt * pl.NB;
  const uint32_t n1 = min(pl.N, n0 + pl.NB);
  const size_t CS = size_t(pl.C) * pl.S;
  const size_t p0 = size_t(c0) * pl.S;

  double acc0[G][W], acc1[G][W], acc2[G][W];
  typename Op::Param prm[G][W];
  bool valid[G];
#pragma unroll
  for (int i = 0; i < G; ++i) {
    const uint32_t j = threadIdx.x + uint32_t(i) * kBlock;
    valid[i] = j < LG;
#pragma unroll
    for (int k = 0; k < W; ++k) {
      acc0[i][k] = acc1[i][k] = acc2[i][k] = 0.0;
      // positions past the tile read channel c0's parameters and are never used
      const uint32_t pos = valid[i] ? j * uint32_t(W) + uint32_t(k) : 0u;
      prm[i][k] = op.load(c0 + div_s.div(pos));
    }
  }

  for (uint32_t n = n0; n < n1; n += uint32_t(STAGES)) {
    V va[STAGES][G], vb[STAGES][G], vc[STAGES][G];
#pragma unroll
    for (int sg = 0; sg < STAGES; ++sg) {
      {
        // unconditional, as in the chunk kernel: a stage past the last sample reads the last sample again, a slot
        // past the tile's end the tile's last group; neither is added below
        const uint32_t ns = (n + uint32_t(sg) < n1) ? n + uint32_t(sg) : n1 - 1u;
        const V *pa = reinterpret_cast<const V *>(a + (size_t(ns) * CS + p0));
        const V *pb = reinterpret_cast<const V *>(b + (size_t(ns) * CS + p0));
        const V *pc = reinterpret_cast<const V *>(c3 + (size_t(ns) * CS + p0));
#pragma unroll
        for (int i = 0; i < G; ++i) {
          const uint32_t j = threadIdx.x + uint32_t(i) * kBlock;
          if (W == 1) {
            // element-aligned arrays (thirty-two 4-byte loads per batch): here the branches cost less than the extra
            // loads do, batch_norm_bwd_var at [1025, 64, 1023] 5.6 TB/s against 4.4
            if (valid[i]) {
              va[sg][i] = load_stream<NT>(&pa[j]);
              if (Op::NIN >= 2) vb[sg][i] = load_stream<NT>(&pb[j]);
              if (Op::NIN >= 3) vc[sg][i] = load_stream<NT>(&pc[j]);
            }
          } else {
            const uint32_t jc = valid[i] ? j : LG - 1u;
            va[sg][i] = load_stream<NT>(&pa[jc]);
            if (Op::NIN >= 2) vb[sg][i] = load_stream<NT>(&pb[jc]);
            if (Op::NIN >= 3) vc[sg][i] = load_stream<NT>(&pc[jc]);
          }
        }
      }
    }
#pragma unroll
    for (int sg = 0; sg < STAGES; ++sg) {
      if (n + uint32_t(sg) < n1) {
#pragma unroll
        for (int i = 0; i < G; ++i) {
          if (valid[i]) {
#pragma unroll
            for (int k = 0; k < W; ++k) {
              chan_reduce_term(op, prm[i][k], lane_get<V>(va[sg][i], k),
                               (Op::NIN >= 2) ? lane_get<V>(vb[sg][i], k) : 0.0f,
                               (Op::NIN >= 3) ? lane_get<V>(vc[sg][i], k) : 0.0f, acc0[i][k], acc1[i][k],
                               acc2[i][k]);
            }
          }
        }
      }
    }
  }

  // fold positions to channels: tpc consecutive lanes share one channel
  uint32_t tpc = 64;
  while (tpc > 1 && tpc * cb > uint32_t(kBlock)) tpc >>= 1;
  const uint32_t cl = threadIdx.x / tpc;
  const uint32_t jj = threadIdx.x % tpc;
  double res[3] = {0.0, 0.0, 0.0};
#pragma unroll
  for (int q = 0; q < Op::NACC; ++q) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < G; ++i) {
      if (valid[i]) {
#pragma unroll
        for (int k = 0; k < W; ++k) {
          lds[tile_slot<P>((threadIdx.x + uint32_t(i) * kBlock) * uint32_t(W) + uint32_t(k))] =
              q == 0 ? acc0[i][k] : (q == 1 ? acc1[i][k] : acc2[i][k]);
        }
      }
    }
    __syncthreads();
    double s = 0.0;
    if (cl < cb) {
      const uint32_t first = cl * pl.S;
      for (uint32_t ss = jj; ss < pl.S; ss += tpc) s += lds[tile_slot<P>(first + ss)];
    }
    res[q] = group_sum(s, int(tpc));
  }
  if (cl < cb && jj == 0) {
    const uint32_t c = c0 + cl;
    if (pl.ppc == 1) {
      op.finalize(c, res[0], res[1], res[2]);
    } else {
      const size_t plane = size_t(pl.C) * pl.ppc;
      const size_t slot = size_t(c) * pl.ppc + nt;
      part[slot] = res[0];
      if (Op::NACC >= 2) part[plane + slot] = res[1];
      if (Op::NACC >= 3) part[2 * plane + slot] = res[2];
    }
  }
}

// "Lane" tiles, for short channels (CB*S positions fit the lanes of one workgroup, 16 bytes per lane): lane t takes
// group t % GPS of sample slot t / GPS, so J = 256 / GPS samples are read side by side and a thread always meets the
// same positions, hence the same channels.  The tile runs over NB samples in steps of J (often all N: then a channel
// has a single partial, nothing goes through the scratch buffer and there is no second kernel).  At the end the
// per-position sums of all J slots meet in LDS and are folded to channels in a fixed order.
template <typename Op, typename V, int NT>
__global__ __launch_bounds__(kBlock) void chan_reduce_lanes_kernel(ReducePlan pl, FastDiv div_s, FastDiv div_g, Op op,
                                                                   const float *__restrict__ a,
                                                                   const float *__restrict__ b,
                                                                   const float *__restrict__ c3,
                                                                   double *__restrict__ part) {
  constexpr int W = VecLanes<V>::n;
  // samples per batch: all loads of a batch are requested before the first is consumed
  // (4, 8 or 16 loads per batch and input measure the same at [49, 2048, 256]: 21.4, 21.6, 22.4 us)
  constexpr int STAGES = Op::NIN == 1 ? 8 : (Op::NIN == 2 ? 4 : 2);
  constexpr uint32_t P = 1024;  // LDS layout of tile_slot: kBlock threads x up to 4 positions
  __shared__ double lds[P + 64];

  const uint32_t nt = blockIdx.x / pl.n_ctiles;
  const uint32_t ct = xcd_contiguous(blockIdx.x % pl.n_ctiles, pl.n_ctiles);
  const uint32_t c0 = ct * pl.CB;
  const uint32_t cb = min(pl.CB, pl.C - c0);
  const uint32_t gps_full = div_g.d;                   // groups per sample of a full tile: the lane pitch of a slot
  const uint32_t gps = (cb * pl.S) / uint32_t(W);      // groups per sample of this tile
  const uint32_t J = pl.J;
  const uint32_t n0 = nt * pl.NB;
  const uint32_t n1 = min(pl.N, n0 + pl.NB);
  const size_t CS = size_t(pl.C) * pl.S;
  uint32_t j, g;
  div_g.divmod(threadIdx.x, j, g);
  const bool active = j < J && g < gps;

  double acc0[W], acc1[W], acc2[W];
  typename Op::Param prm[W];
#pragma unroll
  for (int k = 0; k < W; ++k) {
    acc0[k] = acc1[k] = acc2[k] = 0.0;
    const uint32_t pos = active ? g * uint32_t(W) + uint32_t(k) : 0u;  // idle lanes read channel c0's parameters
    prm[k] = op.load(c0 + div_s.div(pos));
  }

  if (active) {
    const size_t off = size_t(c0) * pl.S + size_t(g) * W;
    const uint64_t step = uint64_t(J) * uint32_t(STAGES);
    auto request = [&](uint64_t n, V(&va)[STAGES], V(&vb)[STAGES], V(&vc)[STAGES]) {
#pragma unroll
      for (int sg = 0; sg < STAGES; ++sg) {
        const uint64_t nn = n + uint64_t(sg) * J;
        if (nn < n1) {
          const size_t at = size_t(nn) * CS + off;
          va[sg] = load_stream<NT>(reinterpret_cast<const V *>(a + at));
          if (Op::NIN >= 2) vb[sg] = load_stream<NT>(reinterpret_cast<const V *>(b + at));
          if (Op::NIN >= 3) vc[sg] = load_stream<NT>(reinterpret_cast<const V *>(c3 + at));
        }
      }
    };
    auto consume = [&](uint64_t n, const V(&va)[STAGES], const V(&vb)[STAGES], const V(&vc)[STAGES]) {
#pragma unroll
      for (int sg = 0; sg < STAGES; ++sg) {
        const uint64_t nn = n + uint64_t(sg) * J;
        if (nn < n1) {
#pragma unroll
          for (int k = 0; k < W; ++k) {
            chan_reduce_term(op, prm[k], lane_get<V>(va[sg], k), (Op::NIN >= 2) ? lane_get<V>(vb[sg], k) : 0.0f,
                             (Op::NIN >= 3) ? lane_get<V>(vc[sg], k) : 0.0f, acc0[k], acc1[k], acc2[k]);
          }
        }
      }
    };
    // One batch at a time: requesting the next batch before the current one is consumed (twice the loads in
    // flight) changes nothing (20.1 us either way for batch_mean at [49, 2048, 256] with unconditional, clamped
    // requests; 31 us with the requests behind branches).
    V va[STAGES], vb[STAGES], vc[STAGES];
    for (uint64_t n = uint64_t(n0) + j; n < n1; n += step) {
      request(n, va, vb, vc);
      consume(n, va, vb, vc);
    }
  }

  // fold (slot, position) to channels: tpc consecutive lanes share one channel and walk its J*S sums, slot by slot
  uint32_t tpc = 64;
  while (tpc > 1 && tpc * cb > uint32_t(kBlock)) tpc >>= 1;
  const uint32_t cl = threadIdx.x / tpc;
  const uint32_t jj = threadIdx.x % tpc;
  const uint32_t per_chan = J * pl.S;
  double res[3] = {0.0, 0.0, 0.0};
#pragma unroll
  for (int q = 0; q < Op::NACC; ++q) {
    __syncthreads();
    if (active) {
#pragma unroll
      for (int k = 0; k < W; ++k) {
        lds[tile_slot<P>(threadIdx.x * uint32_t(W) + uint32_t(k))] = q == 0 ? acc0[k] : (q == 1 ? acc1[k] : acc2[k]);
      }
    }
    __syncthreads();
    double s = 0.0;
    if (cl < cb) {
      for (uint32_t e = jj; e < per_chan; e += tpc) {
        uint32_t slot, ss;
        div_s.divmod(e, slot, ss);
        s += lds[tile_slot<P>(slot * gps_full * uint32_t(W) + cl * pl.S + ss)];
      }
    }
    res[q] = group_sum(s, int(tpc));
  }
  if (cl < cb && jj == 0) {
    const uint32_t c = c0 + cl;
    if (pl.ppc == 1) {
      op.finalize(c, res[0], res[1], res[2]);
    } else {
      const size_t plane = size_t(pl.C) * pl.ppc;
      const size_t slot = size_t(c) * pl.ppc + nt;
      part[slot] = res[0];
      if (Op::NACC >= 2) part[plane + slot] = res[1];
      if (Op::NACC >= 3) part[2 * plane + slot] = res[2];
    }
  }
}

// One wave per channel adds the channel's partials: lane l takes partials
// l, l+64, ... in order, then the lanes meet in a butterfly.
template <typename Op>
__global__ __launch_bounds__(kBlock) void chan_reduce_fold_kernel(uint32_t C, uint32_t ppc, Op op,
                                                                  const double *__restrict__ part) {
  const uint32_t c = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  if (c >= C) return;  // uniform per wave
  double s0 = 0.0, s1 = 0.0, s2 = 0.0;
  const double *p0 = part + size_t(c) * ppc;
  const double *p1 = p0 + size_t(C) * ppc;
  const double *p2 = p1 + size_t(C) * ppc;
  // ppc <= 256 here: a lane's (up to) four partials per sum are requested together, then added in order
  if (ppc != 0u) {
    double v0[4], v1[4], v2[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t j = lane + uint32_t(i) * kWave;
      const uint32_t jc = j < ppc ? j : ppc - 1u;
      v0[i] = p0[jc];
      if (Op::NACC >= 2) v1[i] = p1[jc];
      if (Op::NACC >= 3) v2[i] = p2[jc];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (lane + uint32_t(i) * kWave < ppc) {
        s0 += v0[i];
        if (Op::NACC >= 2) s1 += v1[i];
        if (Op::NACC >= 3) s2 += v2[i];
      }
    }
  }
  s0 = wave_sum(s0);
  if (Op::NACC >= 2) s1 = wave_sum(s1);
  if (Op::NACC >= 3) s2 = wave_sum(s2);
  if (lane == 0) op.finalize(c, s0, s1, s2);
}

// The same for channels with many partials: one workgroup per channel, thread t takes partials t, t+256, ...,
// then the workgroup sum.
template <typename Op>
__global__ __launch_bounds__(kBlock) void chan_reduce_fold_block_kernel(uint32_t C, uint32_t ppc, Op op,
                                                                        const double *__restrict__ part) {
  __shared__ double lds[kBlock / kWave];
  const uint32_t c = blockIdx.x;
  double s0 = 0.0, s1 = 0.0, s2 = 0.0;
  const double *p0 = part + size_t(c) * ppc;
  const double *p1 = p0 + size_t(C) * ppc;
  const double *p2 = p1 + size_t(C) * ppc;
  for (uint32_t j = threadIdx.x; j < ppc; j += kBlock) {
    s0 += p0[j];
    if (Op::NACC >= 2) s1 += p1[j];
    if (Op::NACC >= 3) s2 += p2[j];
  }
  s0 = block_sum(s0, lds);
  if (Op::NACC >= 2) s1 = block_sum(s1, lds);
  if (Op::NACC >= 3) s2 = block_sum(s2, lds);
  if (threadIdx.x == 0) op.finalize(c, s0, s1, s2);
}

// Caller-provided partial-sum buffer for launch_chan_reduce (instead of the per-stream cache, which allocates).
struct FixedScratch {
  void *ptr;
  size_t bytes;
};

// Bytes of partial sums a reduction with NACC sums needs for plan `pl` (0 when every channel has one partial).
inline size_t chan_reduce_scratch_bytes(const ReducePlan &pl, int nacc) {
  return pl.ppc > 1 ? size_t(nacc) * pl.C * pl.ppc * sizeof(double) : 0;
}

// Status of launch_chan_reduce.  The reference ABI is void: its entry points drop the status, which is also
// recorded for anode_gpu_take_last_error().
enum ReduceStatus : int {
  kReduceOk = 0,
  kReduceScratchTooSmall = 1,   // the caller-provided buffer cannot hold the partial sums; nothing was enqueued
  kReduceScratchUnavailable = 2 // the per-stream buffer could not be provided; nothing was enqueued
};

// `fixed` (optional) replaces the per-stream scratch cache: with it the call allocates nothing.
template <typename Op>
int launch_chan_reduce(const char *symbol, uint32_t S, uint32_t C, uint32_t N, Op op, const float *a,
                       const float *b, CUstream_st *stream, const float *c = nullptr,
                       const FixedScratch *fixed = nullptr) {
  const uint32_t len = checked_len(S, C, N, symbol);
  hipStream_t s = as_stream(stream);
  if (len == 0) {
    // No element to add, but every channel still gets its finalised value (0/0 = NaN for a mean, the
    // accumulate twins add their term of an empty sum), as in the reference, whose one block per channel
    // always writes its output (e.g. routines_gpu/batch_norm.cu:52-56).
    if (C > 0) {
      const uint32_t waves_per_block = kBlock / kWave;
      chan_reduce_fold_kernel<Op><<<(C + waves_per_block - 1) / waves_per_block, kBlock, 0, s>>>(C, 0, op, nullptr);
      note_launch(symbol);
    }
    return kReduceOk;
  }
  // the reductions only load, and a 16-byte load is as fast from any 4-byte aligned address: arrays that start at
  // any element take the 16-byte tilings
  const bool ptrs_aligned = true;
  const ReducePlan pl = plan_chan_reduce(S, C, N, ptrs_aligned, uint32_t(tuning().reduce_wg_target), Op::NIN);
  if (Op::NIN < 2) b = a;
  if (Op::NIN < 3) c = a;
  const int nt = stream_policy(size_t(len) * sizeof(float), tuning().reduce_nontemporal);

  ScratchLease lease{nullptr, std::unique_lock<std::mutex>(), nullptr};
  double *part = nullptr;
  const size_t need = chan_reduce_scratch_bytes(pl, Op::NACC);
  if (need > 0) {
    if (fixed) {
      if (need > fixed->bytes) return kReduceScratchTooSmall;
      part = static_cast<double *>(fixed->ptr);
    } else {
      lease = acquire_scratch(s, need, symbol);
      if (!lease.ptr) return kReduceScratchUnavailable;
      part = static_cast<double *>(lease.ptr);
    }
  }
  if (pl.whole == 2) {
    const FastDiv div_s(S);
    const FastDiv div_g(uint32_t((uint64_t(pl.CB) * S + (pl.vec ? 3 : 0)) / (pl.vec ? 4 : 1)));
    if (pl.vec) {
      if (nt) {
        chan_reduce_lanes_kernel<Op, f32x4, kNtLoad><<<pl.grid, kBlock, 0, s>>>(pl, div_s, div_g, op, a, b, c, part);
      } else {
        chan_reduce_lanes_kernel<Op, f32x4, 0><<<pl.grid, kBlock, 0, s>>>(pl, div_s, div_g, op, a, b, c, part);
      }
    } else {
      chan_reduce_lanes_kernel<Op, float, 0><<<pl.grid, kBlock, 0, s>>>(pl, div_s, div_g, op, a, b, c, part);
    }
  } else if (pl.whole) {
    const FastDiv div_s(S);
    auto launch_whole = [&](auto tile_positions) {
      constexpr uint32_t P = decltype(tile_positions)::value;
      if (pl.vec) {
        if (nt) {
          chan_reduce_whole_kernel<Op, f32x4, kNtLoad, P><<<pl.grid, kBlock, 0, s>>>(pl, div_s, op, a, b, c, part);
        } else {
          chan_reduce_whole_kernel<Op, f32x4, 0, P><<<pl.grid, kBlock, 0, s>>>(pl, div_s, op, a, b, c, part);
        }
      } else {
        chan_reduce_whole_kernel<Op, float, 0, P><<<pl.grid, kBlock, 0, s>>>(pl, div_s, op, a, b, c, part);
      }
    };
    if (pl.P == 1024) {
      launch_whole(std::integral_constant<uint32_t, 1024>{});
    } else if (pl.P == 2048) {
      launch_whole(std::integral_constant<uint32_t, 2048>{});
    } else {
      launch_whole(std::integral_constant<uint32_t, 4096>{});
    }
  } else {
    if (pl.vec) {
      if (nt) {
        chan_reduce_chunk_kernel<Op, f32x4, kNtLoad><<<pl.grid, kBlock, 0, s>>>(pl, op, a, b, c, part);
      } else {
        chan_reduce_chunk_kernel<Op, f32x4, 0><<<pl.grid, kBlock, 0, s>>>(pl, op, a, b, c, part);
      }
    } else {
      chan_reduce_chunk_kernel<Op, float, 0><<<pl.grid, kBlock, 0, s>>>(pl, op, a, b, c, part);
    }
  }
  note_launch(symbol);
  if (pl.ppc > 1) {
    if (pl.ppc > 256) {  // few channels, long lists of partials (a scalar sum of a large array)
      chan_reduce_fold_block_kernel<Op><<<C, kBlock, 0, s>>>(C, pl.ppc, op, part);
    } else {
      const uint32_t waves_per_block = kBlock / kWave;
      chan_reduce_fold_kernel<Op><<<(C + waves_per_block - 1) / waves_per_block, kBlock, 0, s>>>(C, pl.ppc, op, part);
    }
    note_launch(symbol);
  }
  return kReduceOk;
}

#endif  // __HIPCC__

}  // namespace anode
