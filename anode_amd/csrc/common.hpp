// Shared host/device helpers for the gfx950 kernels: vector types, exact
// division by launch-invariant divisors, wave64 / workgroup reductions,
// launch geometry and the per-stream scratch cache.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <mutex>
#include <type_traits>

// Layout fixed by the reference (routines_gpu/common.cuh:65-66, src/ffi.rs:28-33).
struct KernelConfig {
  uint32_t block_sz;
  uint32_t max_block_ct;
};
struct CUstream_st;

#define ANODE_EXPORT extern "C" __attribute__((visibility("default")))

namespace anode {

constexpr int kWave = 64;    // CDNA wavefront width
constexpr uint32_t kXcds = 8;  // accelerator dies of an MI355X; workgroup i of a launch runs on die i % 8
constexpr int kBlock = 256;  // workgroup size of every kernel here: 4 waves, one per SIMD

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));

static inline hipStream_t as_stream(CUstream_st *s) { return reinterpret_cast<hipStream_t>(s); }

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline bool aligned4(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

// ---------------------------------------------------------------------------
// Exact unsigned division by a divisor fixed at launch (Granlund-Montgomery,
// round-up method): q = (t + ((n - t) >> sh1)) >> sh2 with t = mulhi(m, n).
// Valid for every n in [0, 2^32) and every d in [1, 2^32).
// ---------------------------------------------------------------------------
struct FastDiv {
  uint32_t d, m, sh1, sh2;

  FastDiv() : d(1), m(1), sh1(0), sh2(0) {}
  explicit FastDiv(uint32_t divisor) : d(divisor) {
    uint32_t l = 0;
    while (l < 32 && (uint64_t(1) << l) < divisor) ++l;  // l = ceil(log2 d)
    const uint64_t two_l = uint64_t(1) << l;
    m = uint32_t(((two_l - divisor) << 32) / divisor + 1);
    sh1 = l < 1 ? l : 1;
    sh2 = l < 1 ? 0 : l - 1;
  }

  __host__ __device__ inline uint32_t div(uint32_t n) const {
#if defined(__HIP_DEVICE_COMPILE__)
    const uint32_t t = __umulhi(m, n);
#else
    const uint32_t t = uint32_t((uint64_t(m) * n) >> 32);
#endif
    return (t + ((n - t) >> sh1)) >> sh2;
  }
  __host__ __device__ inline void divmod(uint32_t n, uint32_t &q, uint32_t &r) const {
    q = div(n);
    r = n - q * d;
  }
};

// ---------------------------------------------------------------------------
// Device-side reductions.  Every lane of the wave must take part.
// ---------------------------------------------------------------------------
#if defined(__HIPCC__)

// Streaming accesses.  Bit 0 of NT marks stores, bit 1 marks loads as
// non-temporal (the `nt` cache policy of global_load/global_store): the data is
// touched once, so it should not displace reusable lines.  NT is a template
// parameter on purpose: a run-time choice between an ordinary and a
// non-temporal access to the same address is folded into one ordinary access
// by the compiler.
constexpr int kNtStore = 1, kNtLoad = 2;

// Runs f(std::integral_constant<int, NT>{}) for a policy value chosen at run time (stream_policy()): nothing,
// streaming stores only, or streaming loads and stores.
template <typename F>
inline void with_stream_policy(int nt, F &&f) {
  if (nt == (kNtLoad | kNtStore)) {
    f(std::integral_constant<int, kNtLoad | kNtStore>{});
  } else if (nt == kNtStore) {
    f(std::integral_constant<int, kNtStore>{});
  } else {
    f(std::integral_constant<int, 0>{});
  }
}

// Workgroups go to the 8 XCDs in turn, each with an L2 (and address translation cache) of its own.  Dealing tiles in
// contiguous ranges per XCD -- tile index i of n becomes the (i / 8)-th tile of the range of XCD i % 8 -- keeps
// neighbouring tiles on one XCD.  Where neighbours share 128-byte lines (a tile's run is not a whole number of
// lines: 196 * CB bytes at S = 49) the neighbour's half of a line is then an L2 hit instead of a second fetch from
// memory (FETCH_SIZE 1.14 x the array -> 1.00 x, 21.9 -> 20.3 us, for batch_mean at [49, 2048, 256]).  Of the
// plane-strided n-d kernels the NLL backward gains 4 % inside a softmax + NLL + backward sequence (106 -> 102 us at
// [512K, 19, 8]) while the softmax itself loses 7 % there (it gains 3 % run alone), so only the backward uses it;
// flat maps gain nothing.
__device__ inline uint32_t xcd_contiguous(uint32_t i, uint32_t n) {
  const uint32_t xcd = i % kXcds, turn = i / kXcds;
  const uint32_t per = n / kXcds, rem = n % kXcds;
  return xcd * per + min(xcd, rem) + turn;
}

// Vector accesses to global memory ask for the element's alignment only (4 bytes; ALIGN = 1 for byte arrays): the
// arrays of the ABI are packed views that may start at any element, and a 16-byte access at such an address is the
// same single instruction.  Measured on 822 MB arrays: a copy whose loads lie 4 bytes off a 16-byte boundary runs at
// 6.55 TB/s against 6.65 aligned; streaming STORES off a boundary cost 15 % (5.6 TB/s: a wave's store then covers
// parts of nine 128-byte lines instead of eight whole ones), so the maps peel a head of up to 31 elements to start
// their stores on a 128-byte line and leave only the loads where they lie.
template <int NT, int ALIGN = 4, typename V>
__device__ inline V load_stream(const V *p) {
  typedef V VU __attribute__((aligned(ALIGN)));
  if constexpr ((NT & kNtLoad) != 0) {
    return __builtin_nontemporal_load(reinterpret_cast<const VU *>(p));
  } else {
    return *reinterpret_cast<const VU *>(p);
  }
}

template <int NT, typename V>
__device__ inline void store_stream(V *p, V v) {
  if constexpr ((NT & kNtStore) != 0 && sizeof(V) == 16) {
    // `nt` together with device scope (`sc1`: the line is written through instead of lingering dirty in the XCD's
    // L2): measured 6.72 TB/s against 6.60 TB/s for `nt` alone on an 822 MB copy.  The builtin cannot express the
    // pair, hence the instruction itself; it is an ordinary vector store.
    // The s_nop keeps the following instruction two wait states away: a VALU write to the data registers of a
    // store of more than 8 bytes needs that distance, and the compiler, which inserts it after its own stores,
    // does not look into inline assembly (seen as wrong values stored by a kernel that recomputed the registers
    // for its next store right away).
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
  } else if constexpr ((NT & kNtStore) != 0) {
    typedef V VU __attribute__((aligned(4)));
    __builtin_nontemporal_store(v, reinterpret_cast<VU *>(p));
  } else {
    typedef V VU __attribute__((aligned(4)));
    *reinterpret_cast<VU *>(p) = v;
  }
}

// Elements to peel off the front of an array of `len` 4-byte elements so that what follows starts on a 128-byte
// line (0 to 31, never more than len).  Streaming stores want more than 16-byte alignment: a wave's store of 1 KiB
// that starts 16 bytes into a 64-byte block leaves a partly written block at either end, and such stores, which
// are written through, cost 12-15 % of the bandwidth (255 -> 292 us for batch_norm at [256,64,112,112]); starting
// on a 64-byte boundary is enough, a whole line is as cheap to reach.
static inline uint32_t head_to_align_line(const void *p, uint32_t len) {
  const uint32_t h = uint32_t((128u - (reinterpret_cast<uintptr_t>(p) & 127u)) & 127u) / 4u;
  return h < len ? h : len;
}

// The streaming policy for kernels that cannot choose where their stores start (rows and planes lie where the
// shape puts them): streaming stores only where every output array starts on a 64-byte boundary; otherwise the
// default policy, whose stores are merged in the L2 before they leave ([8,19,512,1024] softmax one element past a
// boundary: 161 us with streaming stores, 131 us without; 115 us on a boundary).
static inline int policy_for_outputs(int nt, const void *out0, const void *out1 = nullptr) {
  if ((reinterpret_cast<uintptr_t>(out0) & 63u) != 0) return 0;
  if (out1 != nullptr && (reinterpret_cast<uintptr_t>(out1) & 63u) != 0) return 0;
  return nt;
}

// Re-dealing a wave's dwords through LDS, for kernels whose narrow side would otherwise move 4 bytes per lane.
// `wave_lds` is the wave's own 256 dwords (16-byte aligned).  Every thread of the workgroup must call (barriers).
//   deal:   lane l holds dwords 4l..4l+3 (one 16-byte load); afterwards out[j] is dword j*64 + l, so that whatever
//           is then computed from out[j] is stored contiguously across the wave;
//   gather: the inverse: lane l holds dword j*64 + l in in[j]; the result is dwords 4l..4l+3 for one 16-byte store.
__device__ inline void wave_deal_dwords(u32x4 v, uint32_t *wave_lds, uint32_t (&out)[4]) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
  *reinterpret_cast<u32x4 *>(wave_lds + lane * 4u) = v;
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) out[j] = wave_lds[uint32_t(j) * kWave + lane];
}
__device__ inline u32x4 wave_gather_dwords(const uint32_t (&in)[4], uint32_t *wave_lds) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
#pragma unroll
  for (int j = 0; j < 4; ++j) wave_lds[uint32_t(j) * kWave + lane] = in[j];
  __syncthreads();
  return *reinterpret_cast<const u32x4 *>(wave_lds + lane * 4u);
}

template <typename T>
__device__ inline T wave_sum(T v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over aligned groups of `width` lanes (width a power of two <= 64).
template <typename T>
__device__ inline T group_sum(T v, int width) {
  for (int off = width >> 1; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

__device__ inline float group_max(float v, int width) {
  for (int off = width >> 1; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Workgroup sum for kBlock threads: wave butterflies, then the per-wave
// results meet in LDS and are added in wave order.  `lds` holds kBlock/kWave
// values.  The result is valid in every thread.  Ends with a barrier, so `lds`
// may be reused at once.
// (WAVES: waves of the workgroup, kBlock / kWave unless a kernel runs larger workgroups.)
template <typename T, int WAVES = kBlock / kWave>
__device__ inline T block_sum(T v, T *lds) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = v;
  __syncthreads();
  T total = lds[0];
#pragma unroll
  for (int w = 1; w < WAVES; ++w) total += lds[w];
  __syncthreads();
  return total;
}

// Workgroup maximum, same contract as block_sum.
template <int WAVES = kBlock / kWave>
__device__ inline float block_max(float v, float *lds) {
  v = wave_max(v);
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = v;
  __syncthreads();
  float top = lds[0];
#pragma unroll
  for (int w = 1; w < WAVES; ++w) top = fmaxf(top, lds[w]);
  __syncthreads();
  return top;
}

#endif  // __HIPCC__

// ---------------------------------------------------------------------------
// Host runtime (runtime.hip)
// ---------------------------------------------------------------------------

// Compute units of the current device (cached per device).
int device_cu_count();

// Tunable launch parameters; defaults are set in runtime.hip and may be
// changed at run time through anode_gpu_set_tuning() (a test and measurement
// hook, not part of the operator ABI).  Each knob is an atomic read with
// relaxed order, so that a host thread may change one while others launch.
struct Knob {
  std::atomic<int> v;
  operator int() const { return v.load(std::memory_order_relaxed); }
};
struct Tuning {
  Knob flat_wg_per_cu;     // workgroups per CU of a streaming map; 0 = one 16-byte group per thread (full grid)
  Knob reduce_wg_target;   // workgroups a per-channel reduction aims to launch
  Knob nontemporal;        // bit 0: non-temporal stores, bit 1: non-temporal loads (streaming maps); 0, 1 or 3
  Knob reduce_nontemporal; // bit 1: non-temporal loads in the reductions
  Knob nt_min_bytes;       // arrays smaller than this keep the default cache policy (they fit the last-level cache)
  Knob reduce_min_tile;    // fewest elements a reduction tile reads (bounds the share of the per-tile epilogue)
  Knob nt_store_min_bytes; // arrays of at least this size are written with streaming stores (never above nt_min_bytes)
  Knob reduce_tile_pos;    // 0: the reductions choose their tile width; 1024, 2048, 4096: forced where S allows
  Knob reduce_lanes;             // 1: short channels (S <= 1024) use lane tiles (samples side by side in a workgroup)
  Knob reduce_single_pass_grid;  // lane tiles: with at least this many channel groups a tile takes all samples
  Knob reduce_lanes_max_ctiles;  // lane tiles: most channel groups (bounds the grid for very many channels)
  Knob reduce_lanes_min_run;     // lane tiles: fewest contiguous floats a tile reads per sample
  Knob nd_xcd_mask;              // n-d softmax kernels that deal pixel groups per XCD: 1 softmax, 2 NLL backward (default), 4 NLL gather
  Knob nd_bwd_flat_max_plane;    // n-d NLL backward: planes of up to this many pixels are walked as a flat array
  Knob nd_pair_ballast;          // KiB of unused LDS per workgroup of the two-lane n-d softmax forward kernel at 17 to 24 classes (caps the workgroups per CU; 0: no cap)
  Knob nd_sample_reg;            // n-d softmax, short planes with more than 32 classes: whole samples in registers (1) or the tile kernels (0)
  Knob nd_colreg;                // n-d softmax, 33 to 512 classes on planes of 128 pixels and more: column tiles in registers (1) or the other kernels (0)
  Knob row_reglds;               // row softmax, rows of whole 16-byte groups held half in LDS, half in registers: 1 for 16385 to 32768 classes, 2 for 32769 to 65536
};

// The streaming mask to use for an array of `bytes` bytes: the load bit of `mask` from nt_min_bytes on, the store
// bit from nt_store_min_bytes on.
int stream_policy(size_t bytes, int mask);
Tuning &tuning();

// Grid size for a grid-stride streaming kernel over `work_items` units of
// per-thread work: enough workgroups to cover the items once, capped at
// flat_wg_per_cu resident workgroups per CU.
uint32_t stream_grid(uint64_t work_items, int items_per_thread);

// Aborts with a message naming `symbol` unless cfg->block_sz is a power of
// two: the contract of the reference's reduction entry points
// (e.g. routines_gpu/batch_norm.cu:68).
void require_pow2_block(const KernelConfig *cfg, const char *symbol);

// dim0*dim1*dim2 as a 32-bit count; aborts with a message when it does not
// fit (the reference's callers guard this: src/ops_gpu.rs:57-61).
uint32_t checked_len(uint64_t a, uint64_t b, uint64_t c, const char *symbol);

// Looks at the thread's HIP error state after a launch (hipPeekAtLastError: the state is left to the caller) and,
// when an error has appeared, records it for anode_gpu_take_last_error() and prints it to stderr.
void note_launch(const char *symbol);
// Records `e` for anode_gpu_take_last_error() and prints "<symbol>: <what>: <error string>".
void note_error(const char *symbol, hipError_t e, const char *what);

// A device buffer private to (current device, stream), grown on demand and
// kept until anode_gpu_release_scratch().  The lease holds that buffer's own lock
// (not a lock of the whole cache): keep it alive until every kernel that uses the
// buffer has been enqueued, so that two host threads sharing a stream cannot
// interleave their launches; threads on other streams or devices are not held up.
// When the buffer cannot be provided (allocation failure, or the stream is being
// captured and would have to allocate) the error is recorded under `symbol`, ptr
// is null and the lock is not held: the caller skips its launch.
struct ScratchLease {
  void *ptr;
  std::unique_lock<std::mutex> lock;
  std::shared_ptr<void> owner;  // keeps the cache entry (and with it the mutex) alive while the lease is
};
ScratchLease acquire_scratch(hipStream_t stream, size_t bytes, const char *symbol);

}  // namespace anode
