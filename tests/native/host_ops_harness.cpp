// Native caller harness: drives the library the way anode's Rust host side
// does -- through the C++ mirror of src/ops_gpu.rs (tests/native/ops_gpu.hpp),
// linked against the STATIC archive libanode_routines_gpu.a -- and re-runs the
// reference's own GPU tests for this path (tests/test_gpu.rs:595-758) plus the
// batch-norm recipe, checked against the CPU oracle.  Test infrastructure.
#include "tests/native/ops_gpu.hpp"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

using namespace anode_host;

extern "C" {
// oracle/anode_oracle.c
void oracle_batch_mean_f64(uint32_t, uint32_t, uint32_t, const float *, double *);
void oracle_batch_var_f64(uint32_t, uint32_t, uint32_t, float, const float *, const float *, double *);
void oracle_batch_norm_f64(uint32_t, uint32_t, uint32_t, const float *, const float *, const float *, double *);
void oracle_batch_norm_bwd_f64(uint32_t, uint32_t, uint32_t, const float *, const float *, const float *, double *, int);
void oracle_batch_norm_bwd_mean_f64(uint32_t, uint32_t, uint32_t, const float *, const float *, const float *, double *, int);
void oracle_batch_norm_bwd_var_f64(uint32_t, uint32_t, uint32_t, const float *, const float *, const float *, const float *,
                                   const float *, double *, int);
void oracle_batch_var_bwd_f64(uint32_t, uint32_t, uint32_t, const float *, const float *, const float *, const float *,
                              double *, int);
void oracle_batch_var_bwd_mean_f64(uint32_t, uint32_t, uint32_t, const float *, const float *, const float *, const float *,
                                   double *, int);
void oracle_batch_mean_bwd_f64(uint32_t, uint32_t, uint32_t, const float *, const float *, double *, int);
void oracle_softmax_f64(uint32_t, uint32_t, const float *, double *);
}

static int g_checks = 0, g_failed = 0;

#define HIP_OK(x)                                                                       \
  do {                                                                                  \
    hipError_t e_ = (x);                                                                \
    if (e_ != hipSuccess) {                                                             \
      std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);        \
      std::exit(2);                                                                     \
    }                                                                                   \
  } while (0)

static void check(bool ok, const char *what) {
  ++g_checks;
  if (!ok) {
    ++g_failed;
    std::printf("FAIL %s\n", what);
  } else {
    std::printf("ok   %s\n", what);
  }
  std::fflush(stdout);
}

template <typename T>
struct Dev {
  T *p = nullptr;
  size_t n = 0;
  explicit Dev(size_t count) : n(count) { HIP_OK(hipMalloc(&p, (count ? count : 1) * sizeof(T))); }
  Dev(const std::vector<T> &h) : Dev(h.size()) { HIP_OK(hipMemcpy(p, h.data(), n * sizeof(T), hipMemcpyHostToDevice)); }
  ~Dev() { (void)hipFree(p); }
  std::vector<T> host(hipStream_t s) const {
    HIP_OK(hipStreamSynchronize(s));
    std::vector<T> h(n);
    HIP_OK(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
    return h;
  }
};

static bool close_to(const std::vector<float> &got, const std::vector<double> &ref, double rel, double floor) {
  if (got.size() != ref.size()) return false;
  for (size_t i = 0; i < got.size(); ++i) {
    if (std::isnan(ref[i]) != std::isnan(got[i])) return false;
    if (std::isnan(ref[i])) continue;
    if (std::fabs(double(got[i]) - ref[i]) > rel * std::fabs(ref[i]) + floor) {
      std::printf("  element %zu: got %.9g ref %.9g\n", i, double(got[i]), ref[i]);
      return false;
    }
  }
  return true;
}

static float frand(uint32_t &state) {  // small LCG -> roughly N(0,1) by summing uniforms
  float acc = 0.0f;
  for (int i = 0; i < 12; ++i) {
    state = state * 1664525u + 1013904223u;
    acc += float(state >> 8) * (1.0f / 16777216.0f);
  }
  return acc - 6.0f;
}

int main() {
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));  // default priority, non-null stream: what conn.cuda_stream() hands out
  GPUDeviceConn conn;
  conn.stream = stream;
  conn.cfg = KernelConfig{1024, 1024};

  // ---- tests/test_gpu.rs:595-613  test_gpu_op_softmax: zeros[32, 1] -> every p == 1.0/32.0 ----
  for (uint32_t block_sz : {1024u, 8u}) {  // 8 < 32 sends the call to the deterministic entry point (ops_gpu.rs:6153)
    conn.cfg.block_sz = block_sz;
    Dev<float> x(std::vector<float>(32, 0.0f)), y(32);
    auto xa = obatch1d(x.p, 32, 1), ya = obatch1d(y.p, 32, 1);
    SoftmaxOp::apply(WriteCap::Assign, conn, xa, ya);
    bool all = true;
    for (float v : y.host(stream)) all = all && (v == 1.0f / 32.0f);
    check(all, block_sz == 1024 ? "softmax zeros == 1/32 (block entry point)" : "softmax zeros == 1/32 (deterministic entry point)");
  }
  conn.cfg.block_sz = 1024;

  // ---- tests/test_gpu.rs:615-690  softmax_cat_nll, labels [12,17] and [12,42] ----
  {
    Dev<float> x(std::vector<float>(64, 0.0f)), p(64), nll(2);
    Dev<uint32_t> lab(std::vector<uint32_t>{12, 17});
    auto xa = obatch1d(x.p, 32, 2), pa = obatch1d(p.p, 32, 2), na = obatch1d(nll.p, 1, 2);
    auto la = obatch1d(lab.p, 1, 2);
    softmax_categorical_nll(conn, xa, la, pa, na);
    bool all = true;
    for (float v : p.host(stream)) all = all && (v == 1.0f / 32.0f);
    check(all, "softmax_cat_nll: p == 1/32");
    auto h = nll.host(stream);
    check(std::fabs(h[0] - 3.4657359f) < 1e-6f && std::fabs(h[1] - 3.4657359f) < 1e-6f, "softmax_cat_nll: nll == log 32");
    Dev<uint32_t> bad(std::vector<uint32_t>{12, 42});
    auto ba = obatch1d(bad.p, 1, 2);
    SoftmaxCategoricalNLLOp::apply(WriteCap::Assign, conn, pa, ba, na);
    h = nll.host(stream);
    check(std::isfinite(h[0]) && std::isnan(h[1]) && std::isnan(h[0] + h[1]), "softmax_cat_nll: out-of-bounds label -> NaN");
    // tests/test_gpu.rs:692-736: adjoint of the batch sum: dx = 1/32 - [k == label]
    Dev<float> dy(std::vector<float>{1.0f, 1.0f}), dx(64);
    auto dya = obatch1d(dy.p, 1, 2), dxa = obatch1d(dx.p, 32, 2);
    SoftmaxCategoricalNLLBwdOp::apply(WriteCap::Assign, conn, dya, pa, la, dxa);
    auto g = dx.host(stream);
    all = true;
    for (int i = 0; i < 2; ++i)
      for (int k = 0; k < 32; ++k) all = all && (g[k + 32 * i] == 1.0f / 32.0f - float(k == (i == 0 ? 12 : 17)));
    check(all, "softmax_cat_nll adjoint: dx == 1/32 - onehot");
    // accumulate into the same adjoint: doubles it
    SoftmaxCategoricalNLLBwdOp::apply(WriteCap::Accumulate, conn, dya, pa, la, dxa);
    auto g2 = dx.host(stream);
    all = true;
    for (size_t i = 0; i < g.size(); ++i) all = all && (g2[i] == g[i] + g[i]);
    check(all, "softmax_cat_nll adjoint: Accumulate adds into dx");
  }

  // ---- tests/test_gpu.rs:738-758  test_gpu_op_dequantize: ones[32,32,3,1] -> 1.0/255.0 ----
  {
    Dev<uint8_t> x(std::vector<uint8_t>(32 * 32 * 3, 1));
    Dev<float> y(32 * 32 * 3);
    auto xa = obatch3d(x.p, 32, 32, 3, 1);
    auto ya = obatch3d(y.p, 32, 32, 3, 1);
    DequantizeOp::apply(WriteCap::Assign, conn, 0.0f, 1.0f, xa, ya);
    bool all = true;
    for (float v : y.host(stream)) all = all && (v == 1.0f / 255.0f);
    check(all, "dequantize ones == 1/255");
  }

  // ---- batch-norm recipe and its adjoint on [W=7, H=5, C=3, N=4] ----
  {
    const uint32_t W = 7, H = 5, C = 3, N = 4, S = W * H;
    const size_t n = size_t(S) * C * N;
    uint32_t seed = 1;
    std::vector<float> hx(n), hdy(n);
    for (auto &v : hx) v = 2.0f + 3.0f * frand(seed);
    for (auto &v : hdy) v = frand(seed);
    Dev<float> x(hx), dy(hdy), y(n), dx(n), mean(C), var(C), dmean(C), dvar(C);
    auto xa = obatch3d(x.p, W, H, C, N), dya = obatch3d(dy.p, W, H, C, N), ya = obatch3d(y.p, W, H, C, N);
    auto dxa = obatch3d(dx.p, W, H, C, N);
    auto ma = array1d(mean.p, C), va = array1d(var.p, C), dma = array1d(dmean.p, C), dva = array1d(dvar.p, C);
    const float eps = 1e-5f;
    batch_normalize(conn, eps, xa, ma, va, ya);
    batch_normalize_adjoint(conn, dya, xa, ma, va, dma, dva, dxa);
    auto hm = mean.host(stream), hv = var.host(stream), hy = y.host(stream), hdx = dx.host(stream);

    std::vector<double> rm(C), rv(C), ry(n), d1(n), d2(n), d3(n), dm1(C), dm2(C), dvr(C);
    oracle_batch_mean_f64(S, C, N, hx.data(), rm.data());
    oracle_batch_var_f64(S, C, N, eps, hx.data(), hm.data(), rv.data());
    oracle_batch_norm_f64(S, C, N, hx.data(), hm.data(), hv.data(), ry.data());
    check(close_to(hm, rm, 1e-5, 0), "batch_normalize: mean");
    check(close_to(hv, rv, 1e-5, 0), "batch_normalize: var (+eps)");
    check(close_to(hy, ry, 1e-5, 1e-6), "batch_normalize: y");
    oracle_batch_norm_bwd_f64(S, C, N, hdy.data(), hv.data(), nullptr, d1.data(), 0);
    oracle_batch_norm_bwd_mean_f64(S, C, N, hdy.data(), hv.data(), nullptr, dm1.data(), 0);
    oracle_batch_norm_bwd_var_f64(S, C, N, hdy.data(), hx.data(), hm.data(), hv.data(), nullptr, dvr.data(), 0);
    std::vector<float> fdv(C), fdm(C);
    for (uint32_t c = 0; c < C; ++c) fdv[c] = float(dvr[c]);
    oracle_batch_var_bwd_f64(S, C, N, fdv.data(), hx.data(), hm.data(), nullptr, d2.data(), 0);
    oracle_batch_var_bwd_mean_f64(S, C, N, fdv.data(), hx.data(), hm.data(), nullptr, dm2.data(), 0);
    for (uint32_t c = 0; c < C; ++c) fdm[c] = float(dm1[c] + dm2[c]);
    oracle_batch_mean_bwd_f64(S, C, N, fdm.data(), nullptr, d3.data(), 0);
    std::vector<double> rdx(n);
    for (size_t i = 0; i < n; ++i) rdx[i] = d1[i] + d2[i] + d3[i];
    check(close_to(hdx, rdx, 1e-5, 2e-6), "batch_normalize adjoint: dx (assign, accumulate, accumulate)");
    check(close_to(dvar.host(stream), dvr, 1e-5, 1e-7), "batch_normalize adjoint: dvar");
  }

  // ---- failure behaviour: what is unimplemented!() in the reference throws here ----
  {
    Dev<float> x(16), m(2);
    auto xa = obatch3d(x.p, 2, 2, 2, 2);
    auto ma = array1d(m.p, 2);
    bool threw = false;
    try {
      BatchMeanOp::apply(WriteCap::Accumulate, conn, xa, ma);  // src/ops_gpu.rs:3781
    } catch (const Unimplemented &) {
      threw = true;
    }
    check(threw, "BatchMeanOp with WriteCap::Accumulate is unimplemented");
    threw = false;
    xa.packed = false;
    try {
      BatchMeanOp::apply(WriteCap::Assign, conn, xa, ma);  // src/ops_gpu.rs:3784
    } catch (const Unimplemented &) {
      threw = true;
    }
    check(threw, "non-packed input is unimplemented");
  }

  // ---- in-place ReLU and its in-place backward (src/ops_gpu.rs:7906-7940) ----
  {
    std::vector<float> hx = {-2.0f, -0.0f, 0.0f, 0.5f, 3.0f, -1.0f, 7.0f, -8.0f, 1.0f};
    std::vector<float> hd = {1, 2, 3, 4, 5, 6, 7, 8, 9};
    Dev<float> x(hx), d(hd);
    auto xa = array1d(x.p, hx.size()), da = array1d(d.p, hd.size());
    PositiveClipFlatMap::apply_gpu_flat_map_inplace(xa, conn);
    PositiveClipFlatMapBwd::apply_gpu_flat_map_bwd_inplace(da, xa, conn);
    auto y = x.host(stream), g = d.host(stream);
    bool ok = true;
    for (size_t i = 0; i < hx.size(); ++i) {
      const float want_y = hx[i] * float(hx[i] > 0.0f);
      ok = ok && (y[i] == want_y) && (std::signbit(y[i]) == std::signbit(want_y)) && (g[i] == hd[i] * float(want_y > 0.0f));
    }
    check(ok, "positive_clip in place, and its backward in place");
  }

  // ---- running statistics (tests/test_gpu.rs:561-593): 0 -> 0.25 -> 0.4375 at rate 0.25 towards 1 ----
  {
    Dev<float> x(std::vector<float>(1024, 1.0f)), y(std::vector<float>(1024, 0.0f));
    auto xa = array1d(x.p, 1024), ya = array1d(y.p, 1024);
    OnlineAverageOp::apply(conn, 0.25f, xa, ya);
    auto h1 = y.host(stream);
    OnlineAverageOp::apply(conn, 0.25f, xa, ya);
    auto h2 = y.host(stream);
    bool ok = true;
    for (size_t i = 0; i < 1024; ++i) ok = ok && h1[i] == 0.25f && h2[i] == 0.4375f;
    check(ok, "online_average: 0.25 then 0.4375");
    OnlineAddOp::apply(conn, 0.5f, xa, ya);
    auto h3 = y.host(stream);
    ok = true;
    for (size_t i = 0; i < 1024; ++i) ok = ok && h3[i] == 0.9375f;
    check(ok, "online_add: y + 0.5 * x");
  }

  // ---- batch sum / broadcast / per-sample division / fills (src/ops_gpu.rs:7478-7614, 9575-9605, 1244, 2080) ----
  {
    const size_t batch = 10, inner = 37;
    Dev<float> ones(batch), total(1), spread(batch);
    auto oa = array1d(ones.p, batch), ta = array1d(total.p, 1), sa = array1d(spread.p, batch);
    set_constant(conn, 1.0f, oa);
    BatchSumOp::apply(WriteCap::Assign, conn, oa, ta);
    check(total.host(stream)[0] == 10.0f, "batch_sum of ten ones == 10 (the sum the reference's sum-join test expects)");
    BatchSumOp::apply(WriteCap::Accumulate, conn, oa, ta);
    check(total.host(stream)[0] == 20.0f, "batch_sum Accumulate adds");
    BatchBroadcastOp::apply(WriteCap::Assign, conn, ta, sa);
    BatchBroadcastOp::apply(WriteCap::Accumulate, conn, ta, sa);
    auto hs = spread.host(stream);
    bool ok = true;
    for (float v : hs) ok = ok && v == 40.0f;
    check(ok, "batch broadcast: Assign then Accumulate");

    std::vector<float> hx(inner * batch), hr(batch);
    uint32_t seed = 99u;
    for (auto &v : hx) v = frand(seed);
    for (size_t b = 0; b < batch; ++b) hr[b] = 0.5f + float(b);
    Dev<float> x(hx), r(hr), y(inner * batch), nz(inner * batch);
    auto xa = obatch1d(x.p, inner, batch), ra = obatch1d(r.p, 1, batch), ya = obatch1d(y.p, inner, batch);
    FlatBroadcastRdivOp::apply(WriteCap::Assign, conn, xa, ra, ya);
    auto hy = y.host(stream);
    ok = true;
    for (size_t b = 0; b < batch; ++b)
      for (size_t a = 0; a < inner; ++a) ok = ok && hy[a + inner * b] == hx[a + inner * b] / hr[b];
    check(ok, "flat broadcast rdiv: x / r[batch]");
    bool threw = false;
    try {
      FlatBroadcastRdivOp::apply(WriteCap::Accumulate, conn, xa, ra, ya);
    } catch (const Unimplemented &) {
      threw = true;
    }
    check(threw, "FlatBroadcastRdivOp with WriteCap::Accumulate is unimplemented");
    hx[3] = 0.0f;
    hx[5] = -0.0f;
    Dev<float> x2(hx);
    auto x2a = obatch1d(x2.p, inner, batch), nza = obatch1d(nz.p, inner, batch);
    IsNonzeroOp::apply(WriteCap::Assign, conn, x2a, nza);
    auto hn = nz.host(stream);
    ok = true;
    for (size_t i = 0; i < hx.size(); ++i) ok = ok && hn[i] == float(hx[i] != 0.0f);
    check(ok, "is_nonzero");
  }

  check(anode_gpu_take_last_error() == 0, "no launch error recorded");
  HIP_OK(hipStreamDestroy(stream));
  std::printf("%s: %d checks, %d failed\n", g_failed ? "FAILED" : "ALL PASS", g_checks, g_failed);
  return g_failed ? 1 : 0;
}
