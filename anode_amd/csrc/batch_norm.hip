// Batch-norm forward and backward pieces over a packed [S, C, N] array
// (S = dim0 spatial positions, fastest; C = dim1 channels; N = dim2 samples):
// the memory of a contiguous NCHW / NCDHW tensor.
//
// Statistics (mean, var, the three backward reductions) go through the tiled
// fp64 reducer of chan_reduce.hpp; the per-element pieces go through the
// channel-indexed 16-byte map of chan_map.hpp.  Per-channel finalisation is
// done in fp64 and rounded to fp32 once.
#include "chan_map.hpp"
#include "chan_reduce.hpp"
#include "common.hpp"

namespace anode {
namespace {

// ---------------------------------------------------------------------------
// reductions
// ---------------------------------------------------------------------------

struct NoParam {};

__device__ inline void write_out(float *out, uint32_t c, double v, bool accumulate) {
  out[c] = accumulate ? float(double(out[c]) + v) : float(v);
}

// batch_norm.cu:24-57   mean[c] = (sum x) / n
struct MeanReduce {
  static constexpr int NIN = 1, NACC = 1;
  typedef NoParam Param;
  float *mean;
  double n;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ void term(const Param &, float a, float, double &s0, double &, double &) const { s0 += double(a); }
  __device__ void finalize(uint32_t c, double s0, double, double) const { mean[c] = float(s0 / n); }
};

// batch_norm.cu:125-163   var[c] = sum (x - mean[c])^2 / n + eps
struct VarReduce {
  static constexpr int NIN = 1, NACC = 1;
  typedef double Param;
  const float *mean;
  float *var;
  double n, eps;
  __device__ Param load(uint32_t c) const { return double(mean[c]); }
  __device__ void term(const Param &m, float a, float, double &s0, double &, double &) const {
    const double d = double(a) - m;
    s0 = fma(d, d, s0);
  }
  __device__ void finalize(uint32_t c, double s0, double, double) const { var[c] = float(s0 / n + eps); }
};

// batch_norm.cu:240-280   dmean[c] (=|+=) (sum (x - mean[c]) * (-2 dvar[c])) / n
struct VarBwdMeanReduce {
  static constexpr int NIN = 1, NACC = 1;
  typedef double Param;
  const float *dvar, *mean;
  float *dmean;
  double n;
  bool accumulate;
  __device__ Param load(uint32_t c) const { return double(mean[c]); }
  __device__ void term(const Param &m, float a, float, double &s0, double &, double &) const { s0 += double(a) - m; }
  __device__ void finalize(uint32_t c, double s0, double, double) const {
    write_out(dmean, c, s0 * (-2.0 * double(dvar[c])) / n, accumulate);
  }
};

// batch_norm.cu:408-444   dmean[c] (=|+=) sum dy * (-rsqrt(var[c]))
struct NormBwdMeanReduce {
  static constexpr int NIN = 1, NACC = 1;
  typedef NoParam Param;
  const float *var;
  float *dmean;
  bool accumulate;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ void term(const Param &, float a, float, double &s0, double &, double &) const { s0 += double(a); }
  __device__ void finalize(uint32_t c, double s0, double, double) const {
    write_out(dmean, c, -s0 / sqrt(double(var[c])), accumulate);
  }
};

// batch_norm.cu:476-515   dvar[c] (=|+=) sum dy * (x - mean[c]) * (-0.5 * rsqrt(v) / v)
struct NormBwdVarReduce {
  static constexpr int NIN = 2, NACC = 1;  // a = dy, b = x
  typedef double Param;
  const float *mean, *var;
  float *dvar;
  bool accumulate;
  __device__ Param load(uint32_t c) const { return double(mean[c]); }
  __device__ void term(const Param &m, float a, float b, double &s0, double &, double &) const {
    s0 = fma(double(a), double(b) - m, s0);
  }
  __device__ void finalize(uint32_t c, double s0, double, double) const {
    const double v = double(var[c]);
    write_out(dvar, c, s0 * (-0.5 / (sqrt(v) * v)), accumulate);
  }
};

// batch_norm.cu:551-587   dvar[c] (=|+=) sum -dy * y * 0.5 / var[c]
struct NormBwdVarV2Reduce {
  static constexpr int NIN = 2, NACC = 1;  // a = dy, b = y
  typedef NoParam Param;
  const float *var;
  float *dvar;
  bool accumulate;
  __device__ Param load(uint32_t) const { return Param{}; }
  __device__ void term(const Param &, float a, float b, double &s0, double &, double &) const {
    s0 = fma(double(a), double(b), s0);
  }
  __device__ void finalize(uint32_t c, double s0, double, double) const {
    write_out(dvar, c, s0 * (-0.5 / double(var[c])), accumulate);
  }
};

// ---------------------------------------------------------------------------
// per-element pieces.  fp32 arithmetic in the reference's order; 1/sqrt with
// correctly rounded sqrt and divide stands in for CUDA's rsqrtf.  With
// -ffp-contract=off only the fmaf() written here is fused.
// ---------------------------------------------------------------------------

// batch_norm.cu:314-336   y = (x - mean[c]) * rsqrt(var[c])
struct NormMap {
  const float *mean, *var;
  struct Param { float m, rs; };
  __device__ Param load(uint32_t c) const { return Param{mean[c], 1.0f / sqrtf(var[c])}; }
  __device__ float value(const Param &p, float x, float, uint32_t) const { return (x - p.m) * p.rs; }
  __device__ float accum(const Param &p, float x, float, uint32_t, float old) const { return old + (x - p.m) * p.rs; }
};

// batch_norm.cu:354-376   dx (=|+=) dy * rsqrt(var[c])
struct NormBwdMap {
  const float *var;
  struct Param { float rs; };
  __device__ Param load(uint32_t c) const { return Param{1.0f / sqrtf(var[c])}; }
  __device__ float value(const Param &p, float dy, float, uint32_t) const { return dy * p.rs; }
  __device__ float accum(const Param &p, float dy, float, uint32_t, float old) const { return fmaf(dy, p.rs, old); }
};

// batch_norm.cu:181-206   dx (=|+=) dvar[c] * (x - mean[c]) * 2 / n
struct VarBwdMap {
  const float *dvar, *mean;
  float norm;
  struct Param { float dv, m; };
  __device__ Param load(uint32_t c) const { return Param{dvar[c], mean[c]}; }
  __device__ float value(const Param &p, float x, float, uint32_t) const { return p.dv * (x - p.m) * 2.0f / norm; }
  __device__ float accum(const Param &p, float x, float, uint32_t, float old) const { return old + value(p, x, 0.0f, 0u); }
};

// batch_norm.cu:73-95   dx (=|+=) dmean[c] / n
struct MeanBwdMap {
  const float *dmean;
  float norm;
  struct Param { float v; };
  __device__ Param load(uint32_t c) const { return Param{dmean[c] / norm}; }
  __device__ float value(const Param &p, float, float, uint32_t) const { return p.v; }
  __device__ float accum(const Param &p, float, float, uint32_t, float old) const { return old + p.v; }
};

inline double count_of(uint32_t d0, uint32_t d2) { return double(d0) * double(d2); }
// batch_norm.cu:34: the reference forms n as an fp32 product
inline float norm_of(uint32_t d0, uint32_t d2) { return float(d0) * float(d2); }

}  // namespace
}  // namespace anode

using namespace anode;

ANODE_EXPORT void anode_gpu_batch_mean_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                      const float *x, float *mean, const KernelConfig *cfg,
                                                      CUstream_st *stream) {
  require_pow2_block(cfg, __func__);
  launch_chan_reduce(__func__, dim0, dim1, dim2, MeanReduce{mean, count_of(dim0, dim2)}, x, nullptr, stream);
}

ANODE_EXPORT void anode_gpu_batch_mean_bwd_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                          const float *dmean, float *dx, const KernelConfig *,
                                                          CUstream_st *stream) {
  launch_chan_map<0, false>(__func__, dim0, dim1, dim2, MeanBwdMap{dmean, norm_of(dim0, dim2)}, nullptr, nullptr, dx, stream);
}

ANODE_EXPORT void anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                                     const float *dmean, float *dx,
                                                                     const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<0, true>(__func__, dim0, dim1, dim2, MeanBwdMap{dmean, norm_of(dim0, dim2)}, nullptr, nullptr, dx, stream);
}

ANODE_EXPORT void anode_gpu_batch_var_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, float epsilon,
                                                     const float *x, const float *mean, float *var,
                                                     const KernelConfig *cfg, CUstream_st *stream) {
  require_pow2_block(cfg, __func__);
  launch_chan_reduce(__func__, dim0, dim1, dim2, VarReduce{mean, var, count_of(dim0, dim2), double(epsilon)}, x,
                     nullptr, stream);
}

ANODE_EXPORT void anode_gpu_batch_var_bwd_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                         const float *dvar, const float *x, const float *mean,
                                                         float *dx, const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, false>(__func__, dim0, dim1, dim2, VarBwdMap{dvar, mean, norm_of(dim0, dim2)}, x, nullptr, dx, stream);
}

ANODE_EXPORT void anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                                    const float *dvar, const float *x,
                                                                    const float *mean, float *dx,
                                                                    const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, true>(__func__, dim0, dim1, dim2, VarBwdMap{dvar, mean, norm_of(dim0, dim2)}, x, nullptr, dx, stream);
}

ANODE_EXPORT void anode_gpu_batch_var_bwd_mean_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                              const float *dvar, const float *x, const float *mean,
                                                              float *dmean, const KernelConfig *cfg,
                                                              CUstream_st *stream) {
  require_pow2_block(cfg, __func__);
  launch_chan_reduce(__func__, dim0, dim1, dim2, VarBwdMeanReduce{dvar, mean, dmean, count_of(dim0, dim2), false}, x,
                     nullptr, stream);
}

ANODE_EXPORT void anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1,
                                                                         uint32_t dim2, const float *dvar,
                                                                         const float *x, const float *mean,
                                                                         float *dmean, const KernelConfig *cfg,
                                                                         CUstream_st *stream) {
  require_pow2_block(cfg, __func__);
  launch_chan_reduce(__func__, dim0, dim1, dim2, VarBwdMeanReduce{dvar, mean, dmean, count_of(dim0, dim2), true}, x,
                     nullptr, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *x,
                                                      const float *mean, const float *var, float *y,
                                                      const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, false>(__func__, dim0, dim1, dim2, NormMap{mean, var}, x, nullptr, y, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_bwd_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                          const float *dy, const float *var, float *dx,
                                                          const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, false>(__func__, dim0, dim1, dim2, NormBwdMap{var}, dy, nullptr, dx, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_bwd_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                                     const float *dy, const float *var, float *dx,
                                                                     const KernelConfig *, CUstream_st *stream) {
  launch_chan_map<1, true>(__func__, dim0, dim1, dim2, NormBwdMap{var}, dy, nullptr, dx, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_bwd_mean_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                               const float *dy, const float *var, float *dmean,
                                                               const KernelConfig *cfg, CUstream_st *stream) {
  require_pow2_block(cfg, __func__);
  launch_chan_reduce(__func__, dim0, dim1, dim2, NormBwdMeanReduce{var, dmean, false}, dy, nullptr, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_bwd_mean_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1,
                                                                          uint32_t dim2, const float *dy,
                                                                          const float *var, float *dmean,
                                                                          const KernelConfig *cfg,
                                                                          CUstream_st *stream) {
  require_pow2_block(cfg, __func__);
  launch_chan_reduce(__func__, dim0, dim1, dim2, NormBwdMeanReduce{var, dmean, true}, dy, nullptr, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_bwd_var_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                              const float *dy, const float *x, const float *mean,
                                                              const float *var, float *dvar,
                                                              const KernelConfig *cfg, CUstream_st *stream) {
  require_pow2_block(cfg, __func__);
  launch_chan_reduce(__func__, dim0, dim1, dim2, NormBwdVarReduce{mean, var, dvar, false}, dy, x, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_bwd_var_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1,
                                                                         uint32_t dim2, const float *dy,
                                                                         const float *x, const float *mean,
                                                                         const float *var, float *dvar,
                                                                         const KernelConfig *cfg,
                                                                         CUstream_st *stream) {
  require_pow2_block(cfg, __func__);
  launch_chan_reduce(__func__, dim0, dim1, dim2, NormBwdVarReduce{mean, var, dvar, true}, dy, x, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_bwd_var_v2_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2,
                                                                 const float *dy, const float *y, const float *var,
                                                                 float *dvar, const KernelConfig *cfg,
                                                                 CUstream_st *stream) {
  require_pow2_block(cfg, __func__);
  launch_chan_reduce(__func__, dim0, dim1, dim2, NormBwdVarV2Reduce{var, dvar, false}, dy, y, stream);
}

ANODE_EXPORT void anode_gpu_batch_norm_bwd_var_v2_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1,
                                                                            uint32_t dim2, const float *dy,
                                                                            const float *y, const float *var,
                                                                            float *dvar, const KernelConfig *cfg,
                                                                            CUstream_st *stream) {
  require_pow2_block(cfg, __func__);
  launch_chan_reduce(__func__, dim0, dim1, dim2, NormBwdVarV2Reduce{var, dvar, true}, dy, y, stream);
}
