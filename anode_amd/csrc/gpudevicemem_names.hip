// The five entry points that anode calls by their gpudevicemem link names, directly over FFI
// (src/ops_gpu.rs:7486-7505 batch sum, :7595-7614 and :7706-7725 batch broadcast, :9592-9600 broadcast division),
// forwarded to this library's implementations of the same arithmetic.
//
// They live in a translation unit of their own on purpose: in the static archive this object is only pulled in
// while one of these names is still undefined, so a link that also carries a real gpudevicemem (listed first)
// keeps gpudevicemem's definitions and never sees these.
#include "common.hpp"

extern "C" {
void anode_gpu_sum_packed_deterministic_f32(uint32_t, const float *, float *, const KernelConfig *, CUstream_st *);
void anode_gpu_sum_packed_accumulate_deterministic_f32(uint32_t, const float *, float *, const KernelConfig *,
                                                       CUstream_st *);
void anode_gpu_bcast_packed_f32(uint32_t, const float *, float *, const KernelConfig *, CUstream_st *);
void anode_gpu_bcast_packed_accumulate_f32(uint32_t, const float *, float *, const KernelConfig *, CUstream_st *);
void anode_gpu_flat_bcast_rdiv_I1ab_I2b_Oab_packed_f32(uint32_t, uint32_t, const float *, const float *, float *,
                                                       const KernelConfig *, CUstream_st *);
}

// src/ops_gpu.rs:7486-7492: (len, x, y, cfg, stream); y[0] = sum_i x[i]
ANODE_EXPORT void gpudevicemem_sum_packed_deterministic_f32(uint32_t len, const float *x, float *y,
                                                            const KernelConfig *cfg, CUstream_st *stream) {
  anode_gpu_sum_packed_deterministic_f32(len, x, y, cfg, stream);
}

// src/ops_gpu.rs:7499-7505: y[0] += sum_i x[i]
ANODE_EXPORT void gpudevicemem_sum_packed_accumulate_deterministic_f32(uint32_t len, const float *x, float *y,
                                                                       const KernelConfig *cfg,
                                                                       CUstream_st *stream) {
  anode_gpu_sum_packed_accumulate_deterministic_f32(len, x, y, cfg, stream);
}

// src/ops_gpu.rs:7595-7601, :7706-7712: (len of y, x, y, cfg, stream); y[i] = x[0]
ANODE_EXPORT void gpudevicemem_bcast_packed_f32(uint32_t len, const float *x, float *y, const KernelConfig *cfg,
                                                CUstream_st *stream) {
  anode_gpu_bcast_packed_f32(len, x, y, cfg, stream);
}

// src/ops_gpu.rs:7608-7614, :7719-7725: y[i] += x[0]
ANODE_EXPORT void gpudevicemem_bcast_packed_accumulate_f32(uint32_t len, const float *x, float *y,
                                                           const KernelConfig *cfg, CUstream_st *stream) {
  anode_gpu_bcast_packed_accumulate_f32(len, x, y, cfg, stream);
}

// src/ops_gpu.rs:9592-9600: (inner, outer, x, rdivisor, y, cfg, stream); y[a,b] = x[a,b] / rdivisor[b]
ANODE_EXPORT void gpudevicemem_flat_bcast_rdiv_I1ab_I2b_Oab_packed_f32(uint32_t inner_dim, uint32_t outer_dim,
                                                                       const float *x, const float *rdivisor,
                                                                       float *y, const KernelConfig *cfg,
                                                                       CUstream_st *stream) {
  anode_gpu_flat_bcast_rdiv_I1ab_I2b_Oab_packed_f32(inner_dim, outer_dim, x, rdivisor, y, cfg, stream);
}
