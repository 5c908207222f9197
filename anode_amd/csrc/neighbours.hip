// The small kernels either side of the path that anode takes from its sibling
// library gpudevicemem (fills, copy/add, scalar broadcast, batch sum, division by
// a per-sample scalar, running-statistics updates).  The signatures follow the
// call sites in src/ops_gpu.rs; their arithmetic is the closed form the call
// sites imply.
#include "chan_map.hpp"
#include "chan_reduce.hpp"
#include "common.hpp"

namespace anode {
namespace {

struct NoParam {};

// y = x   /   y += x
struct AddMap {
  typedef NoParam Param;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ float value(const Param &, float a, float, uint32_t) const { return a; }
  __device__ float accum(const Param &, float a, float, uint32_t, float old) const { return old + a; }
};
// y = x   /   y *= x
struct MultMap {
  typedef NoParam Param;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ float value(const Param &, float a, float, uint32_t) const { return a; }
  __device__ float accum(const Param &, float a, float, uint32_t, float old) const { return old * a; }
};
// y = rate * x   /   y = fma(rate, x, y)
struct OnlineAddMap {
  float rate;
  typedef NoParam Param;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ float value(const Param &, float a, float, uint32_t) const { return rate * a; }
  __device__ float accum(const Param &, float a, float, uint32_t, float old) const { return fmaf(rate, a, old); }
};
// y = fma(rate, y, x): the running value is discounted, then the new one added
struct OnlineDiscountMap {
  float rate;
  typedef NoParam Param;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ float value(const Param &, float a, float, uint32_t) const { return a; }
  __device__ float accum(const Param &, float a, float, uint32_t, float old) const { return fmaf(rate, old, a); }
};
struct IsNonzeroMap {
  typedef NoParam Param;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ float value(const Param &, float a, float, uint32_t) const { return float(a != 0.0f); }
  __device__ float accum(const Param &, float a, float, uint32_t, float old) const { return old + float(a != 0.0f); }
};
// y = c   /   y += c
struct ConstMap {
  float c;
  typedef NoParam Param;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ float value(const Param &, float, float, uint32_t) const { return c; }
  __device__ float accum(const Param &, float, float, uint32_t, float old) const { return old + c; }
};
// y[i] = x[0]   /   y[i] += x[0]: the scalar lives on the device
struct BcastScalarMap {
  const float *x;
  struct Param { float v; };
  __device__ Param load(uint32_t) const { return Param{x[0]}; }
  __device__ float value(const Param &p, float, float, uint32_t) const { return p.v; }
  __device__ float accum(const Param &p, float, float, uint32_t, float old) const { return old + p.v; }
};
// y[a,b] = x[a,b] / r[b]: a true division per element
struct BcastRdivMap {
  const float *r;
  struct Param { float v; };
  __device__ Param load(uint32_t c) const { return Param{r[c]}; }
  __device__ float value(const Param &p, float a, float, uint32_t) const { return a / p.v; }
  __device__ float accum(const Param &p, float a, float, uint32_t, float old) const { return old + a / p.v; }
};

// y[0] = sum x   /   y[0] += sum x, summed in fp64 in a fixed order
struct ScalarSumReduce {
  static constexpr int NIN = 1, NACC = 1;
  typedef NoParam Param;
  float *y;
  bool accumulate;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ void term(const Param &, float a, float, double &s0, double &, double &) const { s0 += double(a); }
  __device__ void finalize(uint32_t c, double s0, double, double) const {
    y[c] = accumulate ? y[c] + float(s0) : float(s0);
  }
};

}  // namespace
}  // namespace anode

using namespace anode;

ANODE_EXPORT void anode_gpu_sum_packed_deterministic_f32(uint32_t len, const float *x, float *y, const KernelConfig *,
                                                         CUstream_st *stream) {
  if (len == 0) {  // the empty sum still defines y
    launch_chan_map<0, false>(__func__, 1, 1, 1, ConstMap{0.0f}, nullptr, nullptr, y, stream);
    return;
  }
  launch_chan_reduce(__func__, len, 1, 1, ScalarSumReduce{y, false}, x, nullptr, stream);
}

ANODE_EXPORT void anode_gpu_sum_packed_accumulate_deterministic_f32(uint32_t len, const float *x, float *y,
                                                                    const KernelConfig *, CUstream_st *stream) {
  launch_chan_reduce(__func__, len, 1, 1, ScalarSumReduce{y, true}, x, nullptr, stream);
}

ANODE_EXPORT void anode_gpu_bcast_packed_f32(uint32_t len, const float *x, float *y, const KernelConfig *,
                                             CUstream_st *stream) {
  launch_chan_map<0, false>(__func__, len, 1, 1, BcastScalarMap{x}, nullptr, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_bcast_packed_accumulate_f32(uint32_t len, const float *x, float *y, const KernelConfig *,
                                                        CUstream_st *stream) {
  launch_chan_map<0, true>(__func__, len, 1, 1, BcastScalarMap{x}, nullptr, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_flat_bcast_rdiv_I1ab_I2b_Oab_packed_f32(uint32_t inner_dim, uint32_t outer_dim,
                                                                    const float *x, const float *rdivisor, float *y,
                                                                    const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, false>(__func__, inner_dim, outer_dim, 1, BcastRdivMap{rdivisor}, x, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_set_constant_packed_f32(uint32_t len, float c, float *y, const KernelConfig *,
                                                    CUstream_st *stream) {
  launch_chan_map<0, false>(__func__, len, 1, 1, ConstMap{c}, nullptr, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_add_packed_f32(uint32_t len, const float *x, float *y, const KernelConfig *,
                                           CUstream_st *stream) {
  launch_chan_map<1, true>(__func__, len, 1, 1, AddMap{}, x, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_mult_packed_f32(uint32_t len, const float *x, float *y, const KernelConfig *,
                                            CUstream_st *stream) {
  launch_chan_map<1, true>(__func__, len, 1, 1, MultMap{}, x, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_is_nonzero_packed_f32(uint32_t len, const float *x, float *y, const KernelConfig *,
                                                  CUstream_st *stream) {
  launch_chan_map<1, false>(__func__, len, 1, 1, IsNonzeroMap{}, x, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_online_add_packed_f32(uint32_t len, float rate, const float *x, float *y,
                                                  const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, true>(__func__, len, 1, 1, OnlineAddMap{rate}, x, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_online_discount_packed_f32(uint32_t len, float rate, const float *x, float *y,
                                                       const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, true>(__func__, len, 1, 1, OnlineDiscountMap{rate}, x, nullptr, y, stream);
}
