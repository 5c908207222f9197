/*
 * C ABI of the MI355X (gfx950, HIP) implementation of anode's GPU operator
 * library.
 *
 * Part 1 declares the 46 entry points of the reference's
 * routines_gpu/lib.h:32-510 with identical names, parameter order and types,
 * so that anode's Rust bindings (build.rs:61-121 -> src/ffi.rs:35) link
 * against this library unchanged.  Part 2 declares ADDITIVE entry points that
 * have no counterpart in the reference (bindgen ignores them:
 * whitelist_recursively(false), build.rs:63).
 *
 * Conventions shared by every entry point (reference: lib.h:27-39,
 * common.cuh:51-67, src/ops_gpu.rs:670-679):
 *   - all data pointers are DEVICE pointers to packed arrays; they need the
 *     alignment of their element type and nothing more (views that start at
 *     any element of an allocation run the same 16-byte kernels); `cfg` is a
 *     HOST pointer, read during the call;
 *   - `stream` is the runtime's stream handle (a hipStream_t passed through the
 *     opaque struct CUstream_st*; NULL = the null stream);
 *   - the call enqueues work on `stream` and returns; nothing is reported;
 *   - index order is first-index-fastest: element (i0,i1,i2) of a
 *     [dim0,dim1,dim2] array lives at i0 + dim0*(i1 + dim1*i2)
 *     (common.cuh:87-106).  With anode's callers (dim0,dim1,dim2) =
 *     (W*H[*D], C, N), i.e. the memory of a contiguous NCHW / NCDHW tensor;
 *   - dim0*dim1*dim2 must be < 2^32 (src/ops_gpu.rs:57-61);
 *   - `*_accumulate_*` entry points add into the output instead of assigning
 *     (common.cuh:171-193);
 *   - entry points that the reference implements as block reductions abort
 *     the process when cfg->block_sz is not a power of two, as the
 *     reference's host-side assert does (e.g. batch_norm.cu:68).  Otherwise
 *     `cfg` is a hint: launch geometry is chosen by the library.
 */
#ifndef ANODE_ROUTINES_GPU_H_
#define ANODE_ROUTINES_GPU_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Layout fixed by common.cuh:65-66 and the Rust twin in src/ffi.rs:28-33:
 *   struct KernelConfig { uint32_t block_sz; uint32_t max_block_ct; };
 * It is left incomplete here exactly as in lib.h:27; C/C++ callers that need
 * to build one define ANODE_DEFINE_KERNEL_CONFIG before including this file. */
struct KernelConfig;
struct CUstream_st;

#ifdef ANODE_DEFINE_KERNEL_CONFIG
struct KernelConfig {
  uint32_t block_sz;
  uint32_t max_block_ct;
};
#endif

#define ANODE_LAUNCH_TAIL const struct KernelConfig *cfg, struct CUstream_st *stream

/* ===================================================================== */
/* Part 1: the reference ABI                                             */
/* ===================================================================== */

/* ---- batch-norm pieces (batch_norm.cu); n = float(dim0)*float(dim2) ---- */

/* lib.h:32-39, batch_norm.cu:24-71.  mean[c] = (sum_{i0,i2} x) / n */
void anode_gpu_batch_mean_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *x, float *mean, ANODE_LAUNCH_TAIL);
/* lib.h:40-47, batch_norm.cu:73-109.  dx = dmean[c] / n */
void anode_gpu_batch_mean_bwd_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dmean, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:48-55, batch_norm.cu:111-123.  dx += dmean[c] / n */
void anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dmean, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:56-65, batch_norm.cu:125-179.  var[c] = sum (x-mean[c])^2 / n + epsilon (biased; epsilon inside) */
void anode_gpu_batch_var_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, float epsilon, const float *x, const float *mean, float *var, ANODE_LAUNCH_TAIL);
/* lib.h:66-75, batch_norm.cu:181-222.  dx = dvar[c] * (x-mean[c]) * 2 / n */
void anode_gpu_batch_var_bwd_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dvar, const float *x, const float *mean, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:76-85, batch_norm.cu:224-238.  dx += ... */
void anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dvar, const float *x, const float *mean, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:86-95, batch_norm.cu:240-296.  dmean[c] = (sum (x-mean[c]) * (-2*dvar[c])) / n */
void anode_gpu_batch_var_bwd_mean_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dvar, const float *x, const float *mean, float *dmean, ANODE_LAUNCH_TAIL);
/* lib.h:96-105, batch_norm.cu:298-312.  dmean[c] += ... */
void anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dvar, const float *x, const float *mean, float *dmean, ANODE_LAUNCH_TAIL);
/* lib.h:106-115, batch_norm.cu:314-352.  y = (x-mean[c]) * rsqrt(var[c])   (var already holds +epsilon) */
void anode_gpu_batch_norm_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *x, const float *mean, const float *var, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:116-124, batch_norm.cu:354-391.  dx = dy * rsqrt(var[c]) */
void anode_gpu_batch_norm_bwd_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dy, const float *var, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:125-133, batch_norm.cu:393-406.  dx += ... */
void anode_gpu_batch_norm_bwd_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dy, const float *var, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:134-142, batch_norm.cu:408-459.  dmean[c] = sum dy * (-rsqrt(var[c])) */
void anode_gpu_batch_norm_bwd_mean_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dy, const float *var, float *dmean, ANODE_LAUNCH_TAIL);
/* lib.h:143-151, batch_norm.cu:461-474.  dmean[c] += ... */
void anode_gpu_batch_norm_bwd_mean_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dy, const float *var, float *dmean, ANODE_LAUNCH_TAIL);
/* lib.h:152-162, batch_norm.cu:476-532.  dvar[c] = sum dy * (x-mean[c]) * (-0.5 * rsqrt(v) / v), v = var[c] */
void anode_gpu_batch_norm_bwd_var_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dy, const float *x, const float *mean, const float *var, float *dvar, ANODE_LAUNCH_TAIL);
/* lib.h:163-173, batch_norm.cu:534-549.  dvar[c] += ... */
void anode_gpu_batch_norm_bwd_var_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dy, const float *x, const float *mean, const float *var, float *dvar, ANODE_LAUNCH_TAIL);
/* lib.h:174-183, batch_norm.cu:551-603.  dvar[c] = sum -dy * y * 0.5 / var[c]   (from the normalised output y) */
void anode_gpu_batch_norm_bwd_var_v2_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dy, const float *y, const float *var, float *dvar, ANODE_LAUNCH_TAIL);
/* lib.h:184-193, batch_norm.cu:605-619.  dvar[c] += ... */
void anode_gpu_batch_norm_bwd_var_v2_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dy, const float *y, const float *var, float *dvar, ANODE_LAUNCH_TAIL);

/* ---- casts, quantisation, discrete ---- */

/* lib.h:253-258, cast.cu:23-42.  y[i] = (uint32_t) x[i] */
void anode_gpu_upcast_u8_packed_u32(uint32_t len, const uint8_t *x, uint32_t *y, ANODE_LAUNCH_TAIL);
/* lib.h:262-269, discrete.cu:21-60.  y[i0,k,i2] = (x[i0 + dim0*i2] == k) ? 1 : 0 */
void anode_gpu_discrete_one_hot_3d1_packed_f32(uint32_t dim0, uint32_t cat_dim1, uint32_t dim2, const uint32_t *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:397-404, quantize.cu:23-47.  y = fma(float(x), (hi-lo)/255, lo) */
void anode_gpu_dequantize_u8_packed_f32(uint32_t len, float lo, float hi, const uint8_t *x, float *y, ANODE_LAUNCH_TAIL);

/* ---- smooth F1 loss (f1.cu) ---- */

/* lib.h:273-282, f1.cu:23-87.  y[k,n] = -(2*sum_i0 x*t + eps) / (sum_i0 (x+t) + eps) */
void anode_gpu_smooth_negative_f1_loss_3d1_packed_f32(uint32_t dim0, uint32_t cat_dim1, uint32_t dim2, float epsilon, const float *x, const float *target, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:283-293, f1.cu:89-132.  dx = dy[k,n] * -(2 t (t+eps) - eps) / (x+t+eps)^2 */
void anode_gpu_smooth_negative_f1_loss_3d1_bwd_packed_f32(uint32_t dim0, uint32_t cat_dim1, uint32_t dim2, float epsilon, const float *dy, const float *x, const float *target, float *dx, ANODE_LAUNCH_TAIL);

/* ---- flat_join.cu ---- */

/* lib.h:296-302, flat_join.cu:28-60.  y = x1 * float(x2 > 0) */
void anode_gpu_M1_copy_map_M2_unit_step_map_R_product_reduce_flat_join_f32(uint32_t len, const float *x1, const float *x2, float *y, ANODE_LAUNCH_TAIL);

/* ---- flat_map.cu: y[i] = f(x[i]); backward maps dx[i] = g(dy[i], y[i]).
 *      Output may alias the same-index input (in-place ReLU,
 *      src/ops_gpu.rs:7906-7940). ---- */

/* lib.h:305-311, flat_map.cu:44-52,96-106.  m = float(x>0); y = (m + (1-m)*c) * x */
void anode_gpu_leaky_relu_flat_map_f32(uint32_t len, float c, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:312-319, flat_map.cu:60-69,108-119.  m = float(y>0); dx = (m + (1-m)*c) * dy */
void anode_gpu_leaky_relu_flat_map_bwd_f32(uint32_t len, float c, const float *dy, const float *y, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:320-325, flat_map.cu:121-127,348-357.  y = x */
void anode_gpu_copy_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:326-331, flat_map.cu:135-141,359-368.  y = |x| */
void anode_gpu_modulus_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:332-337, flat_map.cu:143-150,370-379.  y = x*x */
void anode_gpu_square_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:338-343, flat_map.cu:158-164,381-390.  y = sqrt(x), correctly rounded */
void anode_gpu_sqrt_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:344-349, flat_map.cu:172-179,392-401.  y = x * float(x>0)   (ReLU by multiply: x<0 -> -0, -inf -> NaN) */
void anode_gpu_positive_clip_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:350-356, flat_map.cu:187-194,403-413.  dx = dy * float(y>0) */
void anode_gpu_positive_clip_flat_map_bwd_f32(uint32_t len, const float *dy, const float *y, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:357-362, flat_map.cu:202-209,415-424.  y = 1 / (1 + exp(-x)) */
void anode_gpu_logistic_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:363-369, flat_map.cu:217-225,426-436.  dx = dy * y * (1-y) */
void anode_gpu_logistic_flat_map_bwd_f32(uint32_t len, const float *dy, const float *y, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:370-375, flat_map.cu:233-240,438-447.  y = float(x>0) */
void anode_gpu_unit_step_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:376-381, flat_map.cu:286-293,449-458.  y = 0.5 * (1 + erf(x / sqrt 2)) */
void anode_gpu_normal_cdf_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:382-387, flat_map.cu:301-307,460-469.  y = tanh(x) */
void anode_gpu_tanh_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:388-393, flat_map.cu:315-323,471-480.  y = 1 / cosh(x)^2 */
void anode_gpu_rcosh2_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);

/* ---- softmax and categorical NLL (softmax.cu).  Row form: element (k,i) of
 *      a [dim0 classes, dim1 rows] array at k + dim0*i.  N-d form: element
 *      (p,k,n) of [prefix_dim, dim0 classes, dim1] at p + prefix_dim*(k + dim0*n),
 *      labels / dy / nll at p + prefix_dim*n. ---- */

/* lib.h:434-440, softmax.cu:24-78.  Row softmax; the reference requires dim0 <= cfg->block_sz
 * (caller dispatch at src/ops_gpu.rs:6153); this implementation accepts any dim0. */
void anode_gpu_softmax_packed_block_f32(uint32_t dim0, uint32_t dim1, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:441-447, softmax.cu:80-142.  Row softmax, any dim0. */
void anode_gpu_softmax_packed_deterministic_f32(uint32_t dim0, uint32_t dim1, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:448-455, softmax.cu:144-175.  nll[i] = label<dim0 ? -log(softmax[label + dim0*i]) : NaN */
void anode_gpu_softmax_cat_nll_packed_f32(uint32_t dim0, uint32_t dim1, const float *softmax, const uint32_t *cat_data, float *nll, ANODE_LAUNCH_TAIL);
/* lib.h:456-464, softmax.cu:177-210.  dx[k,i] = dy[i] * (softmax[k,i] - float(label[i]==k))   (bad label: unmasked) */
void anode_gpu_softmax_cat_nll_bwd_packed_f32(uint32_t dim0, uint32_t dim1, const float *dy, const float *softmax, const uint32_t *cat_data, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:465-473, softmax.cu:212-225.  dx += ... */
void anode_gpu_softmax_cat_nll_bwd_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, const float *dy, const float *softmax, const uint32_t *cat_data, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:474-481, softmax.cu:227-276.  Channel-axis softmax per pixel.  y may be x (in place), as with the
 * reference's kernel, whose threads read nothing but the pixels they write. */
void anode_gpu_softmax_nd_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:482-490, softmax.cu:278-313.  Per-pixel gather, NaN when label >= dim0. */
void anode_gpu_softmax_nd_cat_nll_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1, const float *softmax, const uint32_t *cat_data, float *nll, ANODE_LAUNCH_TAIL);
/* lib.h:491-500, softmax.cu:315-350.  dx[p,k,n] = dy[p,n] * (softmax - float(label[p,n]==k)) */
void anode_gpu_softmax_nd_cat_nll_bwd_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1, const float *dy, const float *softmax, const uint32_t *cat_data, float *dx, ANODE_LAUNCH_TAIL);
/* lib.h:501-510, softmax.cu:352-366.  dx += ... */
void anode_gpu_softmax_nd_cat_nll_bwd_packed_accumulate_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1, const float *dy, const float *softmax, const uint32_t *cat_data, float *dx, ANODE_LAUNCH_TAIL);

/* ===================================================================== */
/* Part 2: additive entry points (no counterpart in the reference)       */
/* ===================================================================== */

/* ---- declared but never implemented by the reference (commented out in lib.h) ---- */

/* lib.h:197-204 (commented out).  y[i,b] = lx[b] * rx[i,b] over [inner_dim, bcast_dim] */
void anode_gpu_bcast_flat_mult_I1b_I2ab_Oab_packed_f32(uint32_t inner_dim, uint32_t bcast_dim, const float *lx, const float *rx, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:205-213 (commented out).  y[i,b] = fma(lx[b], rx[i,b], shift[b]) */
void anode_gpu_bcast_flat_mult_add_I1b_I2ab_Oab_packed_f32(uint32_t inner_dim, uint32_t bcast_dim, const float *lx, const float *rx, const float *shift, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:214-222 (commented out).  y[i,b,o] = lx[b] * rx[i,b,o] over [inner_dim, bcast_dim, outer_dim] */
void anode_gpu_bcast_flat_mult_I1b_I2abc_Oabc_packed_f32(uint32_t inner_dim, uint32_t bcast_dim, uint32_t outer_dim, const float *lx, const float *rx, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:223-232 (commented out).  y[i,b,o] = fma(lx[b], rx[i,b,o], shift[b]): the per-channel affine (gamma, beta) */
void anode_gpu_bcast_flat_mult_add_I1b_I2abc_Oabc_packed_f32(uint32_t inner_dim, uint32_t bcast_dim, uint32_t outer_dim, const float *lx, const float *rx, const float *shift, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:235-241 (commented out).  y = lx * rx */
void anode_gpu_flat_mult_f32(uint32_t len, const float *lx, const float *rx, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:242-249 (commented out).  y = fma(lx, rx, shift) */
void anode_gpu_flat_mult_add_f32(uint32_t len, const float *lx, const float *rx, const float *shift, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:408-414 (commented out).  y[b] = sum_a x[a,b] */
void anode_gpu_sum_Iab_Ob_packed_deterministic_f32(uint32_t reduce_dim, uint32_t outer_dim, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:415-422 (commented out).  y[b] = sum_{a,c} x[a,b,c] */
void anode_gpu_sum_Iabc_Ob_packed_deterministic_f32(uint32_t reduce_inner_dim, uint32_t mid_dim, uint32_t reduce_outer_dim, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* lib.h:423-430 (commented out).  y[b] = sum_{a,c} x[a,b,c]^2 */
void anode_gpu_square_sum_Iabc_Ob_packed_deterministic_f32(uint32_t reduce_inner_dim, uint32_t mid_dim, uint32_t reduce_outer_dim, const float *x, float *y, ANODE_LAUNCH_TAIL);

/* ---- whitelisted for binding by the reference (build.rs:101-102) but never defined there; functor bodies at
 *      flat_map.cu:242-278 ---- */

/* y = x > 0 ? log(x) : -inf   (NaN -> -inf: the comparison is false) */
void anode_gpu_log_positive_clip_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* y = x > 0 ? 1 / x : 0 */
void anode_gpu_positive_reciprocal_flat_map_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);

/* ---- no counterpart in the reference ---- */

/* Inverse of dequantize: scale = (hi-lo)/255; y = clamp(rint((x-lo)/scale), 0, 255), round half to even, NaN -> 0. */
void anode_gpu_quantize_u8_packed_f32(uint32_t len, float lo, float hi, const float *x, uint8_t *y, ANODE_LAUNCH_TAIL);
/* u8 image normalisation in one pass: y[i,b,o] = fma(scale[b], float(x[i,b,o]), shift[b]). */
void anode_gpu_bcast_dequantize_u8_I1b_I2abc_Oabc_packed_f32(uint32_t inner_dim, uint32_t bcast_dim, uint32_t outer_dim, const float *scale, const float *shift, const uint8_t *x, float *y, ANODE_LAUNCH_TAIL);
/* batch_mean and batch_var in one pass over x: mean[c], var[c] = biased variance + epsilon (composes with batch_norm). */
void anode_gpu_batch_mean_var_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, float epsilon, const float *x, float *mean, float *var, ANODE_LAUNCH_TAIL);
/* The same launch also moves the layer's running statistics (src/ops.rs:1002-1003: online_average of the mean and of
 * var + epsilon): run[c] = fma(rate, stat[c] - run[c], run[c]) on the fp32 values stored in mean and var, so the
 * result equals batch_mean_var followed by two anode_gpu_online_average_packed_f32 launches bit for bit.  Either
 * running array may be null. */
void anode_gpu_batch_mean_var_online_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, float epsilon, float rate, const float *x, float *mean, float *var, float *run_mean, float *run_var, ANODE_LAUNCH_TAIL);
/* batch_mean_var for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  No counterpart in the reference (whose one-block-per-channel reductions need no
 * workspace).  Same kernels, geometry and results as anode_gpu_batch_mean_var_3d1_packed_f32, but the partial sums
 * go to a 4 MiB device array that is part of the library image (one copy per GPU, held until the process ends)
 * instead of the per-stream buffer: the call makes no hipMalloc / hipFree and no allocating library call.  Returns
 * 0, or non-zero with nothing enqueued: 1 = the shape needs more than 4 MiB of partial sums (2 * dim1 * tiles per
 * channel doubles; use the entry point above), 2 = the array's device address could not be obtained, or the call
 * could not be put in order behind the previous one.  All calls on one GPU share the array.  Outside graph capture
 * the library keeps them apart on the device, whatever streams and host threads they come from: every call records an
 * event behind its kernels (created once per device, with the address look-up), and a call on another stream than the
 * previous one waits for it.  A call that is captured takes no part in that: graphs that hold such calls must not be
 * replayed so that they overlap each other, or other calls of this entry point, on one GPU. */
int anode_gpu_batch_mean_var_3d1_packed_noalloc_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, float epsilon, const float *x, float *mean, float *var, ANODE_LAUNCH_TAIL);
/* batch_norm followed by positive_clip in one pass: t = (x-mean[c])*rsqrt(var[c]); y = t * float(t>0). */
void anode_gpu_batch_norm_positive_clip_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *x, const float *mean, const float *var, float *y, ANODE_LAUNCH_TAIL);
/* batch_norm followed by the per-channel affine in one pass: y = fma((x-mean[c])*rsqrt(var[c]), gamma[c], beta[c]). */
void anode_gpu_batch_norm_affine_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *x, const float *mean, const float *var, const float *gamma, const float *beta, float *y, ANODE_LAUNCH_TAIL);
/* The three backward reductions in one pass over (dy, x): dvar = batch_norm_bwd_var; dmean = batch_norm_bwd_mean +
 * batch_var_bwd_mean(dvar).  mask may be NULL; otherwise dy is first multiplied by float(mask>0) (ReLU backward). */
void anode_gpu_batch_norm_bwd_reduce_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dy, const float *x, const float *mean, const float *var, const float *mask, float *dmean, float *dvar, ANODE_LAUNCH_TAIL);
/* The three backward maps in one pass: dx = batch_norm_bwd + batch_var_bwd(dvar) + batch_mean_bwd(dmean), the terms
 * formed and added exactly as the three separate launches do.  mask as above. */
void anode_gpu_batch_norm_bwd_apply_3d1_packed_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dy, const float *x, const float *mean, const float *var, const float *dmean, const float *dvar, const float *mask, float *dx, ANODE_LAUNCH_TAIL);
/* dx += ... */
void anode_gpu_batch_norm_bwd_apply_3d1_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, uint32_t dim2, const float *dy, const float *x, const float *mean, const float *var, const float *dmean, const float *dvar, const float *mask, float *dx, ANODE_LAUNCH_TAIL);
/* Row softmax and softmax_cat_nll in one pass over x (src/ops.rs:1172-1176 as one launch); writes the same softmax and
 * nll as anode_gpu_softmax_packed_*_f32 followed by anode_gpu_softmax_cat_nll_packed_f32 (NaN for a label >= dim0).
 * "The same" is to the bit: the kernel, and with it the order in which a row's exponentials are added, follows the
 * shape alone.  The one exception is rows of more than 32768 classes whose length is not a multiple of four: there
 * the order depends on where a row starts within a 128-byte line of the output, so the two agree to the bit where
 * the arrays of the two calls lie alike (as arrays handed out by an allocator do). */
void anode_gpu_softmax_cat_nll_fused_packed_f32(uint32_t dim0, uint32_t dim1, const float *x, const uint32_t *cat_data, float *softmax, float *nll, ANODE_LAUNCH_TAIL);
/* The same plus anode_gpu_softmax_cat_nll_bwd_packed_f32 in that launch, for a dy that is known before the forward
 * pass (e.g. ones for a summed loss): dx[k,i] = dy[i] * (softmax[k,i] - float(label[i]==k)). */
void anode_gpu_softmax_cat_nll_fused_fwd_bwd_packed_f32(uint32_t dim0, uint32_t dim1, const float *x, const uint32_t *cat_data, const float *dy, float *softmax, float *nll, float *dx, ANODE_LAUNCH_TAIL);
/* softmax_nd and softmax_nd_cat_nll in one pass over x; writes the same softmax and nll as the two entry points. */
void anode_gpu_softmax_nd_cat_nll_fused_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1, const float *x, const uint32_t *cat_data, float *softmax, float *nll, ANODE_LAUNCH_TAIL);
/* The same and the backward pass for a dy known before the forward pass, in one launch: softmax, nll and dx as
 * softmax_nd, softmax_nd_cat_nll and softmax_nd_cat_nll_bwd write them (softmax.cu:227-334), bit for bit. */
void anode_gpu_softmax_nd_cat_nll_fused_fwd_bwd_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1, const float *x, const uint32_t *cat_data, const float *dy, float *softmax, float *nll, float *dx, ANODE_LAUNCH_TAIL);
/* Running statistics: y <- fma(rate, x - y, y) (the semantics of anode's online_average, tests/test_gpu.rs:561-593). */
void anode_gpu_online_average_packed_f32(uint32_t len, float rate, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* Device form of the host rule src/utils/mod.rs:31-41 per row of a [dim0 (fastest), dim1] array: first index of the
 * strict maximum, NaN never selected, 0 when nothing exceeds -inf. */
void anode_gpu_arg_max_packed_u32(uint32_t dim0, uint32_t dim1, const float *x, uint32_t *index, ANODE_LAUNCH_TAIL);

/* "Ignore" variants of the four NLL entry points above: a label >= the number of classes contributes nll = 0 and
 * dx = 0 (dx unchanged for _accumulate) instead of the reference's NaN and unmasked dy*p (softmax.cu:294-296, :331).
 * In-range labels give bit-identical results to the plain entry points. */
void anode_gpu_softmax_cat_nll_ignore_packed_f32(uint32_t dim0, uint32_t dim1, const float *softmax, const uint32_t *cat_data, float *nll, ANODE_LAUNCH_TAIL);
void anode_gpu_softmax_cat_nll_bwd_ignore_packed_f32(uint32_t dim0, uint32_t dim1, const float *dy, const float *softmax, const uint32_t *cat_data, float *dx, ANODE_LAUNCH_TAIL);
void anode_gpu_softmax_cat_nll_bwd_ignore_packed_accumulate_f32(uint32_t dim0, uint32_t dim1, const float *dy, const float *softmax, const uint32_t *cat_data, float *dx, ANODE_LAUNCH_TAIL);
void anode_gpu_softmax_nd_cat_nll_ignore_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1, const float *softmax, const uint32_t *cat_data, float *nll, ANODE_LAUNCH_TAIL);
void anode_gpu_softmax_nd_cat_nll_bwd_ignore_packed_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1, const float *dy, const float *softmax, const uint32_t *cat_data, float *dx, ANODE_LAUNCH_TAIL);
void anode_gpu_softmax_nd_cat_nll_bwd_ignore_packed_accumulate_f32(uint32_t prefix_dim, uint32_t dim0, uint32_t dim1, const float *dy, const float *softmax, const uint32_t *cat_data, float *dx, ANODE_LAUNCH_TAIL);

/* ---- the neighbours anode takes from its sibling library gpudevicemem (source not part of the reference tree) ----
 * Signatures follow the call sites in src/ops_gpu.rs; the arithmetic is the closed form those call sites imply.
 * Exported under this library's prefix; the five that anode calls directly over FFI are repeated below under
 * their gpudevicemem names. */

/* src/ops_gpu.rs:7486-7492 (gpudevicemem_sum_packed_deterministic_f32): y[0] = sum_i x[i]; fp64 accumulation in a fixed order. */
void anode_gpu_sum_packed_deterministic_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:7499-7505.  y[0] += sum_i x[i] */
void anode_gpu_sum_packed_accumulate_deterministic_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:7595-7601 (gpudevicemem_bcast_packed_f32): y[i] = x[0] for i < len; x is a device scalar. */
void anode_gpu_bcast_packed_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:7608-7614.  y[i] += x[0] */
void anode_gpu_bcast_packed_accumulate_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:9592-9600 (gpudevicemem_flat_bcast_rdiv_I1ab_I2b_Oab_packed_f32): y[a,b] = x[a,b] / rdivisor[b]. */
void anode_gpu_flat_bcast_rdiv_I1ab_I2b_Oab_packed_f32(uint32_t inner_dim, uint32_t outer_dim, const float *x, const float *rdivisor, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:1244, :2080 (set_zeros, set_constant): y[i] = c. */
void anode_gpu_set_constant_packed_f32(uint32_t len, float c, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:108, :557 (add): y[i] += x[i].  (copy is anode_gpu_copy_flat_map_f32.) */
void anode_gpu_add_packed_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:3346 (mult): y[i] *= x[i]. */
void anode_gpu_mult_packed_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:3636 (is_nonzero): y[i] = float(x[i] != 0). */
void anode_gpu_is_nonzero_packed_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:5886 (online_add): y[i] = fma(rate, x[i], y[i]). */
void anode_gpu_online_add_packed_f32(uint32_t len, float rate, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:5972, :6015 (online_discount; the momentum buffer of src/ops.rs:1425-1430): y[i] = fma(rate, y[i], x[i]).
 * The arithmetic is read off the name and the momentum recipe; gpudevicemem's kernel is not in the reference tree. */
void anode_gpu_online_discount_packed_f32(uint32_t len, float rate, const float *x, float *y, ANODE_LAUNCH_TAIL);

/* The same five under the link names anode calls them by, directly over FFI, for a build that has no ROCm
 * gpudevicemem yet.  In the static archive they sit in an object of their own (gpudevicemem_names.o), which the
 * linker only pulls in while one of these names is still undefined: list a real gpudevicemem before this library
 * and its definitions win; never force-load (--whole-archive) both. */
/* src/ops_gpu.rs:7486-7492 */
void gpudevicemem_sum_packed_deterministic_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:7499-7505 */
void gpudevicemem_sum_packed_accumulate_deterministic_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:7595-7601, :7706-7712 */
void gpudevicemem_bcast_packed_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:7608-7614, :7719-7725 */
void gpudevicemem_bcast_packed_accumulate_f32(uint32_t len, const float *x, float *y, ANODE_LAUNCH_TAIL);
/* src/ops_gpu.rs:9592-9600 */
void gpudevicemem_flat_bcast_rdiv_I1ab_I2b_Oab_packed_f32(uint32_t inner_dim, uint32_t outer_dim, const float *x, const float *rdivisor, float *y, ANODE_LAUNCH_TAIL);

/* The host-side rule itself (src/utils/mod.rs:31-41), for logits already on the host: first index of the strict
 * maximum starting from (-inf, 0); NaN never selected.  xs is a HOST pointer. */
size_t anode_host_arg_max_f32(const float *xs, size_t len);

/* The reduction scratch.  No reference counterpart: the reference reduces a channel in one block and needs no
 * workspace; this library cuts a channel into tiles and keeps one fp64 partial sum per (channel, tile) in a device
 * buffer per (device, stream), allocated by the first reduction call on that stream and grown on demand.  When the
 * buffer cannot be provided -- allocation failure, or the stream is being captured into a HIP graph and holds no
 * buffer that is large enough -- the reduction entry point enqueues nothing, reports on stderr and records the
 * hipError_t for anode_gpu_take_last_error().  A HIP graph keeps the buffer of the stream it was captured on: graphs
 * captured on one stream must not be replayed concurrently with each other or with eager reduction calls on that
 * stream. */
/* Upper bound of the scratch bytes any reduction entry point needs for a [dim0, dim1, dim2] array, for either
 * alignment of its arrays.  The bound holds for the library's tiling as it is when the function is called: the
 * tiling is fixed for a build and only moves through the library's undeclared measurement hook, after which the
 * query must be repeated. */
size_t anode_gpu_reduce_scratch_bytes(uint32_t dim0, uint32_t dim1, uint32_t dim2);
/* Makes `stream` (current device) hold at least `bytes` of scratch, so that later calls allocate nothing (call it
 * before capturing the stream).  Returns 0 or the hipError_t of the failed allocation. */
int anode_gpu_reserve_scratch(struct CUstream_st *stream, size_t bytes);
/* Frees the scratch of `stream` (current device); the caller has synchronised the stream.  Returns the number of
 * buffers freed. */
int anode_gpu_release_scratch(struct CUstream_st *stream);

/* Library introspection.  No reference counterpart. */
/* 0 when no launch made by this library has failed since the last call; otherwise the hipError_t
 * of the most recent failure.  Reading clears it.  The thread's own HIP error state is never cleared by this library
 * (the reference's kernels leave it to the caller, whose own checks must keep seeing what they see today): a failed
 * launch is noticed by peeking at that state, so while the caller leaves an error pending there (no
 * hipGetLastError()), a later launch that fails with the same hipError_t cannot be told from the pending one and is
 * not recorded again.  Refusals (scratch unavailable, stream under capture) are always recorded. */
int anode_gpu_take_last_error(void);
/* Number of entry points of Part 1 (46). */
uint32_t anode_gpu_reference_symbol_count(void);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* ANODE_ROUTINES_GPU_H_ */
