// Host-side runtime shared by all entry points: device queries, launch
// geometry, the per-(device, stream) scratch cache and error bookkeeping.
#include "chan_reduce.hpp"
#include "common.hpp"

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <utility>
#include <vector>

namespace anode {

namespace {

constexpr int kMaxDevices = 64;
std::atomic<int> g_cu_count[kMaxDevices];
std::atomic<int> g_last_error{0};

// One buffer per (device, stream), each behind a lock of its own: a reduction holds its stream's lock from the
// lookup until both of its kernels are enqueued, so host threads that share a stream cannot interleave their
// launches, while threads on different streams or devices never wait for each other.  The map's own lock is held
// for the lookup only.  Entries are shared_ptrs: anode_gpu_release_scratch() takes an entry out of the map and
// frees its buffers once no lease holds it.
struct ScratchBuf {
  std::mutex mu;
  void *ptr = nullptr;
  size_t cap = 0;
  std::vector<void *> outgrown;  // earlier, smaller buffers: kernels in flight may still use them
};
std::mutex g_scratch_map_mutex;
std::map<std::pair<int, hipStream_t>, std::shared_ptr<ScratchBuf>> g_scratch;

Tuning g_tuning = {
    /*flat_wg_per_cu=*/{{0}},
    /*reduce_wg_target=*/{{8192}},
    /*nontemporal=*/{{3}},
    /*reduce_nontemporal=*/{{2}},
    /*nt_min_bytes=*/{{192 << 20}},
    /*reduce_min_tile=*/{{16384}},
    /*nt_store_min_bytes=*/{{16 << 20}},
    /*reduce_tile_pos=*/{{0}},
    /*reduce_lanes=*/{{1}},
    /*reduce_single_pass_grid=*/{{256}},
    /*reduce_lanes_max_ctiles=*/{{2048}},
    /*reduce_lanes_min_run=*/{{128}},
    /*nd_xcd_mask=*/{{2}},
    /*nd_bwd_flat_max_plane=*/{{131072}},
    /*nd_pair_ballast=*/{{32}},
    /*nd_sample_reg=*/{{1}},
    /*nd_colreg=*/{{1}},
    /*row_reglds=*/{{3}},
    };

}  // namespace

int device_cu_count() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
  int n = g_cu_count[dev].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
    n = 256;  // MI355X
  }
  g_cu_count[dev].store(n, std::memory_order_relaxed);
  return n;
}

Tuning &tuning() { return g_tuning; }

uint32_t stream_grid(uint64_t work_items, int items_per_thread) {
  const uint64_t per_block = uint64_t(kBlock) * uint64_t(items_per_thread > 0 ? items_per_thread : 1);
  uint64_t blocks = (work_items + per_block - 1) / per_block;
  if (g_tuning.flat_wg_per_cu > 0) {
    const uint64_t cap = uint64_t(device_cu_count()) * uint64_t(g_tuning.flat_wg_per_cu);
    if (blocks > cap) blocks = cap;
  }
  if (blocks < 1) blocks = 1;
  return uint32_t(blocks);
}

int stream_policy(size_t bytes, int mask) {
  const size_t load_min = size_t(g_tuning.nt_min_bytes > 0 ? g_tuning.nt_min_bytes : 0);
  size_t store_min = size_t(g_tuning.nt_store_min_bytes > 0 ? g_tuning.nt_store_min_bytes : 0);
  if (store_min > load_min) store_min = load_min;
  int out = 0;
  if (bytes >= load_min) out |= mask & 2;   // kNtLoad
  if (bytes >= store_min) out |= mask & 1;  // kNtStore
  return out;
}

void require_pow2_block(const KernelConfig *cfg, const char *symbol) {
  const uint32_t b = cfg->block_sz;
  if (b == 0 || (b & (b - 1)) != 0) {
    std::fprintf(stderr, "%s: KernelConfig.block_sz = %u is not a power of two\n", symbol, b);
    std::abort();
  }
}

uint32_t checked_len(uint64_t a, uint64_t b, uint64_t c, const char *symbol) {
  // a, b, c < 2^32, so a*b cannot overflow 64 bits; guard the second product.
  const uint64_t ab = a * b;
  if (ab > 0xffffffffull || ab * c > 0xffffffffull) {
    std::fprintf(stderr, "%s: %llu x %llu x %llu elements do not fit a 32-bit index\n", symbol,
                 (unsigned long long)a, (unsigned long long)b, (unsigned long long)c);
    std::abort();
  }
  return uint32_t(ab * c);
}

void note_launch(const char *symbol) {
  // Peek, never take: the thread's HIP error state belongs to the caller (the reference's kernels never touch
  // the CUDA error state, so the host framework's own checks must keep seeing what they see today).  An error
  // that was already pending at this thread's previous check is not reported again.
  static thread_local hipError_t pending = hipSuccess;
  const hipError_t e = hipPeekAtLastError();
  if (e != hipSuccess && e != pending) {
    g_last_error.store(int(e), std::memory_order_relaxed);
    std::fprintf(stderr, "%s: HIP error pending after the launch: %s\n", symbol, hipGetErrorString(e));
  }
  pending = e;
}

void note_error(const char *symbol, hipError_t e, const char *what) {
  g_last_error.store(int(e), std::memory_order_relaxed);
  std::fprintf(stderr, "%s: %s: %s; nothing was enqueued\n", symbol, what, hipGetErrorString(e));
}

namespace {
uint32_t ceil_div_u32(uint64_t a, uint64_t b) { return uint32_t((a + b - 1) / b); }
uint32_t gcd_u32(uint32_t a, uint32_t b) {
  while (b) {
    const uint32_t t = a % b;
    a = b;
    b = t;
  }
  return a;
}
}  // namespace

ReducePlan plan_chan_reduce(uint32_t S, uint32_t C, uint32_t N, bool ptrs_aligned, uint32_t wg_target, int nin) {
  ReducePlan p{};
  p.S = S;
  p.C = C;
  p.N = N;
  if (S == 0 || C == 0 || N == 0) return p;
  const uint64_t total = uint64_t(S) * C * N;
  // elements a tile aims to read: enough tiles to fill the chip, but never so
  // small that the per-tile epilogue dominates
  uint64_t per_tile = total / (wg_target ? wg_target : 1);
  const uint64_t floor_elems = g_tuning.reduce_min_tile > 0 ? uint64_t(g_tuning.reduce_min_tile) : 1;
  if (per_tile < floor_elems) per_tile = floor_elems;

  if (S > kTilePos) {
    p.whole = 0;
    p.CB = 1;
    p.n_ctiles = C;
    p.vec = (ptrs_aligned && S % 4 == 0) ? 1 : 0;
    if (uint64_t(S) >= 2 * per_tile) {
      p.n_stiles = ceil_div_u32(S, per_tile);
      // whole 128-byte lines per tile, so that neighbouring tiles (on different XCDs) never fetch the same line
      p.SB = (ceil_div_u32(S, p.n_stiles) + 31u) & ~31u;
      p.n_stiles = ceil_div_u32(S, p.SB);
      p.NB = 1;
    } else {
      p.n_stiles = 1;
      p.SB = S;
      uint64_t nb = per_tile / S;
      if (nb < 1) nb = 1;
      if (nb > N) nb = N;
      p.NB = uint32_t(nb);
      // a channel of at most 56 steps of a workgroup (1024 floats each) is one tile: no second launch
      // ([12544, 16, 4]: batch_mean + batch_norm_bwd_var 20.4 -> 16.1 us)
      if (uint64_t(N) * ceil_div_u32(S, 1024u) <= 56u) p.NB = N;
    }
  } else {
    p.SB = S;
    p.n_stiles = 1;
    bool vec = ptrs_aligned && (uint64_t(C) * S) % 4 == 0;
    // a tile that is not the whole channel axis must start a whole number of 16-byte groups into the array: CB*S a multiple of 4
    const uint32_t unit = 4 / gcd_u32(S, 4);
    const uint32_t lane_cap = kBlock * (vec ? 4u : 1u);  // positions that one pass of a workgroup's lanes covers
    // (with 16-byte accesses a tile is either the whole channel axis or a multiple of `unit` channels: one of the
    // two must fit the lanes)
    bool lanes = g_tuning.reduce_lanes > 0 && S <= lane_cap &&
                 (!vec || uint64_t(C) * S <= lane_cap || uint64_t(unit) * S <= lane_cap);
    if (lanes) {
      // "lane" tiles: few channels, all (or many) samples, several samples side by side in the workgroup
      uint32_t cb_max = lane_cap / S;
      if (cb_max > kMaxTileChans) cb_max = kMaxTileChans;
      if (cb_max >= C) {
        cb_max = C;
      } else if (vec) {
        cb_max -= cb_max % unit;
      }
      // (with two or more input arrays twice the run: measured 34.5 us against 37.0 us for batch_norm_bwd_var at
      // [49, 2048, 256], while one-input reductions lose 2 us with the longer run)
      const uint32_t run = (g_tuning.reduce_lanes_min_run > 0 ? uint32_t(g_tuning.reduce_lanes_min_run) : 1u) *
                           (nin >= 2 ? 2u : 1u);
      const uint32_t max_ctiles = g_tuning.reduce_lanes_max_ctiles > 0 ? uint32_t(g_tuning.reduce_lanes_max_ctiles) : 1u;
      uint32_t cb = ceil_div_u32(run, S);                 // a sample's run of the tile is at least `run` floats long
      const uint32_t fit = ceil_div_u32(C, max_ctiles);   // and the grid stays bounded
      if (cb < fit) cb = fit;
      if (vec) cb = ceil_div_u32(cb, unit) * unit;
      if (cb > cb_max) cb = cb_max;
      {
        // among the legal widths from there on, the one that keeps most lanes busy (J slots of gps lanes each)
        const uint32_t step = (vec && cb_max != C) ? unit : 1u;
        const uint32_t w = vec ? 4u : 1u;
        uint32_t best = cb, best_busy = 0;
        for (uint32_t k = cb; k <= cb_max && k < cb + 64 * step; k += step) {
          if (vec && k != C && k % unit != 0) continue;
          const uint32_t gps_k = ceil_div_u32(uint64_t(k) * S, w);
          const uint32_t busy = (kBlock / gps_k) * gps_k;
          if (busy > best_busy && ceil_div_u32(C, k) * 2 >= ceil_div_u32(C, cb)) {
            best = k;
            best_busy = busy;
          }
        }
        cb = best;
      }
      p.whole = 2;
      p.CB = cb;
      p.vec = vec ? 1 : 0;
      p.n_ctiles = ceil_div_u32(C, cb);
      const uint32_t gps = ceil_div_u32(uint64_t(cb) * S, vec ? 4u : 1u);  // 16-byte (or 4-byte) groups per sample
      p.J = kBlock / gps;
      // One tile per channel group where there are enough groups to fill the GPU, and also where a group's samples
      // are few steps of the workgroup (at most 64: eight batches of loads): there the second launch costs more than
      // the idle CUs lose ([784, 16, 32] batch_mean 9.6 -> 7.8 us, the nine batch-norm entry points 82 -> 65 us;
      // [784, 16, 128], 128 steps, 12.0 us against 9.9 with sample tiles and the fold kernel).
      if (p.n_ctiles >= uint32_t(g_tuning.reduce_single_pass_grid) || ceil_div_u32(N, p.J) <= 64u) {
        p.NB = N;  // one tile per channel group: no partial sums, no second kernel
      } else {
        uint64_t nb = per_tile / (uint64_t(cb) * S);
        if (nb < p.J) nb = p.J;
        if (nb > N) nb = N;
        p.NB = uint32_t(nb);
      }
    } else {
      p.whole = 1;
      // channels of a tile of P positions, and whether it keeps 16-byte accesses (CB*S a multiple of 4)
      auto fit = [&](uint32_t P, uint32_t &cb_out) {
        uint32_t k = P / S;
        if (k > kMaxTileChans) k = kMaxTileChans;
        if (k > C) k = C;
        bool v = vec && k > 0;
        if (v && k != C) {
          if (k >= unit) {
            k -= k % unit;
          } else {
            v = false;
          }
        }
        cb_out = k;
        return v;
      };
      // the narrowest tile width that keeps 16-byte accesses (where any does) and wastes at most an eighth of
      // its positions; failing that, the widest
      uint32_t P = kTilePos, cb = 0;
      bool any_vec = false;
      for (uint32_t q = kTilePosMin; q <= kTilePos; q <<= 1) {
        uint32_t k;
        any_vec = any_vec || (q >= S && fit(q, k));
      }
      for (uint32_t q = kTilePosMin; q <= kTilePos; q <<= 1) {
        uint32_t k;
        if (q < S) continue;
        const bool v = fit(q, k);
        if (v == any_vec && uint64_t(k) * S * 8 >= uint64_t(q) * 7) {
          P = q;
          break;
        }
      }
      if (g_tuning.reduce_tile_pos >= int(kTilePosMin) && uint32_t(g_tuning.reduce_tile_pos) >= S) {
        P = uint32_t(g_tuning.reduce_tile_pos) >= kTilePos ? kTilePos : (g_tuning.reduce_tile_pos >= 2048 ? 2048u : 1024u);
      }
      vec = fit(P, cb);
      // few channels: a narrower tile holds them just as well
      while (P > kTilePosMin && uint64_t(cb) * S <= P / 2) P >>= 1;
      p.P = P;
      p.CB = cb;
      p.vec = vec ? 1 : 0;
      p.n_ctiles = ceil_div_u32(C, cb);
      uint64_t nb = per_tile / (uint64_t(cb) * S);
      if (nb < 1) nb = 1;
      if (nb > N) nb = N;
      p.NB = uint32_t(nb);
      // a channel group of at most 32 steps of a workgroup (1024 positions each) is one tile, and of at most 64
      // where the channel groups fill the GPU by themselves: no second launch ([3136, 16, 8]: batch_mean +
      // batch_norm_bwd_var 20.4 -> 16.0 us; [3136, 64, 16], 64 steps, 21.6 against 20.3 with two tiles and the fold)
      const uint64_t steps = uint64_t(N) * (P / 1024u);
      if (steps <= 32u || (steps <= 64u && p.n_ctiles >= 256u)) p.NB = N;
    }
  }
  p.n_ntiles = ceil_div_u32(N, p.NB);
  p.NB = ceil_div_u32(N, p.n_ntiles);  // balance the samples over the tiles
  p.n_ntiles = ceil_div_u32(N, p.NB);
  p.ppc = p.n_stiles * p.n_ntiles;
  p.grid = p.n_ctiles * p.n_stiles * p.n_ntiles;
  return p;
}

ScratchLease acquire_scratch(hipStream_t stream, size_t bytes, const char *symbol) {
  int dev = 0;
  (void)hipGetDevice(&dev);
  std::shared_ptr<ScratchBuf> entry;
  {
    std::lock_guard<std::mutex> map_lock(g_scratch_map_mutex);
    std::shared_ptr<ScratchBuf> &slot = g_scratch[std::make_pair(dev, stream)];
    if (!slot) slot = std::make_shared<ScratchBuf>();
    entry = slot;
  }
  ScratchLease lease{nullptr, std::unique_lock<std::mutex>(entry->mu), entry};
  ScratchBuf &buf = *entry;
  if (buf.cap < bytes) {
    // Growing means hipMalloc, which a stream under capture cannot take (it would fail and could invalidate the
    // capture): refuse instead, and tell the caller how to avoid it.  A query that itself fails (no device; the
    // legacy stream while another stream is being captured in global mode) refuses as well: nothing is allocated
    // on a stream whose state is unknown.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    const hipError_t q = hipStreamIsCapturing(stream, &capturing);
    if (q != hipSuccess) {
      note_error(symbol, q, "cannot read the capture state of the stream, so the reduction scratch is not allocated");
      lease.lock.unlock();
      return lease;
    }
    if (capturing != hipStreamCaptureStatusNone) {
      note_error(symbol, hipErrorStreamCaptureUnsupported,
                 "the stream is being captured and has no reduction scratch yet (call anode_gpu_reserve_scratch "
                 "or run the entry point once on this stream before capturing)");
      lease.lock.unlock();
      return lease;
    }
    // Grow geometrically.  The previous buffer may still be read by kernels in flight on this stream, so it is
    // not freed here; anode_gpu_release_scratch() frees everything a stream holds once the caller has
    // synchronised it.
    size_t cap = buf.cap ? buf.cap : size_t(1) << 16;
    while (cap < bytes) cap <<= 1;
    void *p = nullptr;
    const hipError_t e = hipMalloc(&p, cap);
    if (e != hipSuccess || !p) {
      note_error(symbol, e != hipSuccess ? e : hipErrorOutOfMemory, "cannot allocate the reduction scratch");
      lease.lock.unlock();
      return lease;
    }
    if (buf.ptr) buf.outgrown.push_back(buf.ptr);
    buf.ptr = p;
    buf.cap = cap;
  }
  lease.ptr = buf.ptr;
  return lease;
}

}  // namespace anode

ANODE_EXPORT int anode_gpu_take_last_error(void) {
  return anode::g_last_error.exchange(0, std::memory_order_relaxed);
}

ANODE_EXPORT uint32_t anode_gpu_reference_symbol_count(void) { return 46; }

// Upper bound of the partial-sum bytes a reduction over [S, C, N] needs: three sums, either alignment.
ANODE_EXPORT size_t anode_gpu_reduce_scratch_bytes(uint32_t S, uint32_t C, uint32_t N) {
  const uint32_t target = uint32_t(anode::tuning().reduce_wg_target);
  size_t most = 0;
  for (int nin = 1; nin <= 2; ++nin) {
    for (int aligned = 0; aligned <= 1; ++aligned) {
      const size_t b = anode::chan_reduce_scratch_bytes(anode::plan_chan_reduce(S, C, N, aligned != 0, target, nin), 3);
      if (b > most) most = b;
    }
  }
  return most;
}

// Makes sure that the reduction entry points find at least `bytes` of partial-sum scratch for `stream` on the
// current device, so that later calls on that stream allocate nothing (needed before the stream is captured into a
// HIP graph).  Returns 0 or the hipError_t of the failed allocation.
ANODE_EXPORT int anode_gpu_reserve_scratch(CUstream_st *stream, size_t bytes) {
  anode::ScratchLease lease = anode::acquire_scratch(anode::as_stream(stream), bytes, __func__);
  if (lease.ptr || bytes == 0) return 0;
  const int e = anode::g_last_error.load(std::memory_order_relaxed);
  return e ? e : int(hipErrorOutOfMemory);
}

// Frees every scratch buffer held for `stream` on the current device.  The caller must have synchronised the
// stream: kernels in flight would lose their partial sums.  Returns the number of buffers freed.
ANODE_EXPORT int anode_gpu_release_scratch(CUstream_st *stream) {
  int dev = 0;
  (void)hipGetDevice(&dev);
  std::shared_ptr<anode::ScratchBuf> entry;
  {
    std::lock_guard<std::mutex> map_lock(anode::g_scratch_map_mutex);
    const auto it = anode::g_scratch.find(std::make_pair(dev, anode::as_stream(stream)));
    if (it == anode::g_scratch.end()) return 0;
    entry = it->second;
    anode::g_scratch.erase(it);
  }
  if (!entry) return 0;
  std::lock_guard<std::mutex> lock(entry->mu);  // a call that is still enqueueing on this stream finishes first
  int freed = 0;
  for (void *p : entry->outgrown) freed += (hipFree(p) == hipSuccess);
  if (entry->ptr) freed += (hipFree(entry->ptr) == hipSuccess);
  entry->outgrown.clear();
  entry->ptr = nullptr;
  entry->cap = 0;
  return freed;
}

// Host-only view of the reduction tiling for a [S, C, N] array, as 12 words:
// whole, CB, SB, n_ctiles, n_stiles, NB, n_ntiles, ppc, vec, grid, P, J.
ANODE_EXPORT void anode_gpu_plan_reduce(uint32_t S, uint32_t C, uint32_t N, int ptrs_aligned,
                                        uint32_t *out12) {
  // bit 1 of ptrs_aligned set: the plan of a reduction with two or more input arrays
  const anode::ReducePlan p = anode::plan_chan_reduce(S, C, N, (ptrs_aligned & 1) != 0,
                                                      uint32_t(anode::tuning().reduce_wg_target),
                                                      (ptrs_aligned & 2) ? 2 : 1);
  const uint32_t v[12] = {p.whole, p.CB, p.SB, p.n_ctiles, p.n_stiles, p.NB, p.n_ntiles, p.ppc, p.vec, p.grid, p.P, p.J};
  std::memcpy(out12, v, sizeof(v));
}

// Host-only check of the exact-division helper: returns n / d computed the way
// the kernels compute it.
ANODE_EXPORT uint32_t anode_gpu_fastdiv_probe(uint32_t n, uint32_t d) { return anode::FastDiv(d).div(n); }

// Test and measurement hook (not declared in the public header).  Knobs: 0 flat_wg_per_cu, 2 reduce_wg_target,
// 3 nontemporal (0, 1 or 3: streaming loads without streaming stores is not a policy the maps are built for),
// 4 reduce_nontemporal, 5 nt_min_bytes, 6 reduce_min_tile, 7 nt_store_min_bytes, 8 reduce_tile_pos,
// 9 reduce_lanes, 10 reduce_single_pass_grid, 11 reduce_lanes_max_ctiles, 12 reduce_lanes_min_run, 13 nd_xcd_mask,
// 14 nd_bwd_flat_max_plane, 15 row_reglds, 16 nd_pair_ballast, 17 nd_sample_reg,
// 18 nd_colreg.  Returns the previous value; a
// negative value only reads.  Returns -1, and changes nothing, for an unknown knob or a value the knob does not take.
ANODE_EXPORT int anode_gpu_set_tuning(int knob, int value) {
  anode::Tuning &t = anode::tuning();
  anode::Knob *slot = nullptr;
  switch (knob) {
    case 0: slot = &t.flat_wg_per_cu; break;
    case 2: slot = &t.reduce_wg_target; break;
    case 3: slot = &t.nontemporal; break;
    case 4: slot = &t.reduce_nontemporal; break;
    case 5: slot = &t.nt_min_bytes; break;
    case 6: slot = &t.reduce_min_tile; break;
    case 7: slot = &t.nt_store_min_bytes; break;
    case 8: slot = &t.reduce_tile_pos; break;
    case 9: slot = &t.reduce_lanes; break;
    case 10: slot = &t.reduce_single_pass_grid; break;
    case 11: slot = &t.reduce_lanes_max_ctiles; break;
    case 12: slot = &t.reduce_lanes_min_run; break;
    case 13: slot = &t.nd_xcd_mask; break;
    case 14: slot = &t.nd_bwd_flat_max_plane; break;
    case 15: slot = &t.row_reglds; break;
    case 16: slot = &t.nd_pair_ballast; break;
    case 17: slot = &t.nd_sample_reg; break;
    case 18: slot = &t.nd_colreg; break;
    default: return -1;
  }
  if (knob == 3 && value >= 0 && value != 0 && value != 1 && value != 3) return -1;
  const int old = *slot;
  if (value >= 0) slot->v.store(value, std::memory_order_relaxed);
  return old;
}
