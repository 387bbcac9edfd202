// Double-precision entry points (gfx950).  The reference instantiates every kernel
// for double as well (AT_DISPATCH_FLOATING_TYPES_AND_HALF, matmul_cuda_kernel.cu:489
// and on, banded_cuda_kernel.cu:389 and on).  logbmm forward and backward run factored on
// the double-precision matrix instruction (f64_mm.h); the max / prod-max products run tiled
// through LDS and their backward is a scatter (f64_max.h).  Everything else here is the
// reference's algorithm in the plain form - one lane per result cell, the reduction axis
// walked in ascending order, lanes along the contiguous axis so that loads and stores
// coalesce.
#include <cfloat>

#include "banded_cells.h"
#include "f64_max.h"
#include "f64_mm.h"

namespace GENBMM_NS {
namespace {

constexpr double kFloorD = -1e9;

enum { kLog = 0, kMax = 1, kSample = 2, kProdMax = 3 };  // the reference's dense modes

// --------------------------------------------------------------- dense forward
// Reference kernels matmul_cuda_kernel.cu:13-45 (log) and :77-121 (sample): two passes
// (maximum, then sum of exponentials) for the log-sum-exp.
template <int MODE>
__global__ __launch_bounds__(256) void k64_fwd(const double* __restrict__ a,
                                              const double* __restrict__ b,
                                              double* __restrict__ out, int32_t* __restrict__ idx,
                                              uint64_t seed, uint64_t offset, int M, int K, int N,
                                              long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int n = (int)(e % N);
  const long bm = e / N;  // batch*M + m
  const long batch = bm / M;
  const double* arow = a + bm * K;
  const double* bcol = b + batch * K * N + n;
  double m = kFloorD;
  for (int k = 0; k < K; ++k) {
    const double v = arow[k] + bcol[(long)k * N];
    if (v > m) m = v;
  }
  double val = 0.0;
  for (int k = 0; k < K; ++k) val += exp(arow[k] + bcol[(long)k * N] - m);
  const double o = log(val) + m;
  out[e] = o;
  if (MODE == kSample) {
    // inverse CDF in ascending k (:109-118); index 0 when the walk never brackets r.
    // One uniform per cell from the same Philox4x32-10 stream as the float path.
    const double r = (double)philox_uniform((uint64_t)e, seed, offset);
    double acc = 0.0;
    int ind = 0;
    for (int k = 0; k < K; ++k) {
      const double p = exp(arow[k] + bcol[(long)k * N] - o);
      if (acc < r && acc + p > r) {
        ind = k;
        break;
      }
      acc += p;
    }
    idx[e] = ind;
  }
}

// -------------------------------------------------------------- logbmm backward
// grad_b[k,n] = sum_m exp(a[m,k] + b[k,n] - out[m,n]) g[m,n]: one lane per cell,
// lanes along n (reference :190-217, the transposed second call of genmul.py:38-41).
__global__ __launch_bounds__(256) void k64_log_bwd_b(const double* __restrict__ a,
                                                    const double* __restrict__ b,
                                                    const double* __restrict__ out,
                                                    const double* __restrict__ g,
                                                    double* __restrict__ grad_b, int M, int K,
                                                    int N, long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int n = (int)(e % N);
  const long bk = e / N;
  const long batch = bk / K;
  const int k = (int)(bk - batch * K);
  const double bv = b[e];
  const double* acol = a + batch * M * K + k;
  const double* ocol = out + batch * M * N + n;
  const double* gcol = g + batch * M * N + n;
  double acc = 0.0;
  for (int m = 0; m < M; ++m)
    acc = __builtin_fma(exp(acol[(long)m * K] + bv - ocol[(long)m * N]), gcol[(long)m * N], acc);
  grad_b[e] = acc;
}

// grad_a[m,k] = sum_n exp(a[m,k] + b[k,n] - out[m,n]) g[m,n] (reference :159-184).
// One wave per row m: the lanes split n (b, out and g are read along their
// contiguous axis) and the 64 partial sums are added across the wave per k.
__global__ __launch_bounds__(256) void k64_log_bwd_a(const double* __restrict__ a,
                                                    const double* __restrict__ b,
                                                    const double* __restrict__ out,
                                                    const double* __restrict__ g,
                                                    double* __restrict__ grad_a, int M, int K,
                                                    int N, long rows) {
  const int lane = threadIdx.x & 63;
  const long bm = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (bm >= rows) return;  // whole waves leave together
  const long batch = bm / M;
  const double* arow = a + bm * K;
  const double* orow = out + bm * N;
  const double* grow = g + bm * N;
  const double* bb = b + batch * K * N;
  for (int k = 0; k < K; ++k) {
    const double av = arow[k];
    double acc = 0.0;
    for (int n = lane; n < N; n += 64)
      acc = __builtin_fma(exp(av + bb[(long)k * N + n] - orow[n]), grow[n], acc);
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) acc += __shfl_xor(acc, s, 64);
    if (lane == 0) grad_a[bm * K + k] = acc;
  }
}

// ------------------------------------------------------ logbmm second order
// Same closed form as the float kernels: with p = exp(a+b-out), w = u_a + u_b,
//   t = sum_k p w;  grad_a = sum_n g p (w - t);  grad_b = sum_m g p (w - t)
// (reference :220-331 computes them as quartic loops).
struct BB64 {
  const double* a; const double* b; const double* out; const double* g;
  const double* ua; const double* ub;
  double* ga; double* gb; double* gg;
  int M, K, N;
};

__global__ __launch_bounds__(256) void k64_bb_t(const BB64 p, long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int n = (int)(e % p.N);
  const long bm = e / p.N;
  const long batch = bm / p.M;
  const double* arow = p.a + bm * p.K;
  const double* uarow = p.ua ? p.ua + bm * p.K : nullptr;
  const double* bcol = p.b + batch * p.K * p.N + n;
  const double* ubcol = p.ub ? p.ub + batch * p.K * p.N + n : nullptr;
  const double o = p.out[e];
  double t = 0.0;
  for (int k = 0; k < p.K; ++k) {
    const double pr = exp(arow[k] + bcol[(long)k * p.N] - o);
    const double w = (uarow ? uarow[k] : 0.0) + (ubcol ? ubcol[(long)k * p.N] : 0.0);
    t = __builtin_fma(pr, w, t);
  }
  p.gg[e] = t;
}

__global__ __launch_bounds__(256) void k64_bb_a(const BB64 p, long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int k = (int)(e % p.K);
  const long bm = e / p.K;
  const long batch = bm / p.M;
  const double av = p.a[e];
  const double uav = p.ua ? p.ua[e] : 0.0;
  const double* brow = p.b + (batch * p.K + k) * p.N;
  const double* ubrow = p.ub ? p.ub + (batch * p.K + k) * p.N : nullptr;
  const double* orow = p.out + bm * p.N;
  const double* grow = p.g + bm * p.N;
  const double* trow = p.gg + bm * p.N;
  double acc = 0.0;
  for (int n = 0; n < p.N; ++n) {
    const double pr = exp(av + brow[n] - orow[n]);
    const double w = uav + (ubrow ? ubrow[n] : 0.0) - trow[n];
    acc = __builtin_fma(grow[n] * pr, w, acc);
  }
  p.ga[e] = acc;
}

__global__ __launch_bounds__(256) void k64_bb_b(const BB64 p, long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int n = (int)(e % p.N);
  const long bk = e / p.N;
  const long batch = bk / p.K;
  const int k = (int)(bk - batch * p.K);
  const double bv = p.b[e];
  const double ubv = p.ub ? p.ub[e] : 0.0;
  const double* acol = p.a + batch * p.M * p.K + k;
  const double* uacol = p.ua ? p.ua + batch * p.M * p.K + k : nullptr;
  const double* ocol = p.out + batch * p.M * p.N + n;
  const double* gcol = p.g + batch * p.M * p.N + n;
  const double* tcol = p.gg + batch * p.M * p.N + n;
  double acc = 0.0;
  for (int m = 0; m < p.M; ++m) {
    const long mn = (long)m * p.N;
    const double pr = exp(acol[(long)m * p.K] + bv - ocol[mn]);
    const double w = (uacol ? uacol[(long)m * p.K] : 0.0) + ubv - tcol[mn];
    acc = __builtin_fma(gcol[mn] * pr, w, acc);
  }
  p.gb[e] = acc;
}

// ---------------------------------------------------------------- dispatch
template <int MODE>
int run_fwd64(const double* a, const double* b, double* out, int32_t* idx, uint64_t seed,
              uint64_t offset, int B, int M, int K, int N, void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || (MODE != kLog && missing(idx, mn)))
    return GENBMM_E_NULLPTR;
  if (mn == 0) return GENBMM_OK;
  hipLaunchKernelGGL((k64_fwd<MODE>), blocks_for(mn), dim3(256), 0, (hipStream_t)stream, a, b, out,
                     idx, seed, offset, M, K, N, (long)mn);
  return launch_status();
}

// max / prod-max forward: one workgroup per 64 x 64 tile of the result
template <bool PROD>
int run_max_fwd64(const double* a, const double* b, double* out, int32_t* idx, int B, int M, int K, int N,
                  void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(idx, mn)) return GENBMM_E_NULLPTR;
  if (mn == 0) return GENBMM_OK;
  const int tiles_m = ceil_div(M, kD64Tile), tiles_n = ceil_div(N, kD64Tile);
  const int64_t total = (int64_t)B * tiles_m * tiles_n;
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  const int vec_o = (N % 4 == 0) && aligned16(out) && aligned16(idx);
  hipLaunchKernelGGL((k64_max_fwd<PROD>), dim3((unsigned)total), dim3(256), 0, (hipStream_t)stream, a, b, out, idx,
                     M, K, N, tiles_m, tiles_n, vec_o);
  return launch_status();
}

// Parts per workgroup for a reduction axis of K cells: the smallest power of two that covers it,
// at most `most` (2^most parts; 64 lanes in all).
inline int argmax64_parts_shift(int K, int most) {
  int ps = 0;
  while (ps < most && (kArg64 << ps) < K) ++ps;
  return ps;
}

template <bool PROD>
int run_argmax_bwd64(const double* a, const double* b, const int32_t* idx, const double* g,
                     double* grad_a, double* grad_b, int B, int M, int K, int N, void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(idx, mn) || missing(g, mn) || missing(grad_a, mk) || missing(grad_b, kn) ||
      (PROD && (missing(a, mk) || missing(b, kn))))
    return GENBMM_E_NULLPTR;
  if (mk == 0 && kn == 0) return GENBMM_OK;
  // (an empty M or N leaves one gradient without workgroups; the other is then all zeros)
  const int ps_a = argmax64_parts_shift(K, 6);
  const int row_tiles = ceil_div(M, 64 >> ps_a), kc_a = ceil_div(K, kArg64 << ps_a);
  // columns: runs of at least 16 adjacent columns (128 bytes of every row of idx-and-g read)
  const int ps_b = argmax64_parts_shift(K, 2);
  const int col_tiles = ceil_div(N, 64 >> ps_b), kc_b = ceil_div(K, kArg64 << ps_b);
  const int64_t total = (int64_t)B * ((int64_t)row_tiles * kc_a + (int64_t)col_tiles * kc_b);
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  hipLaunchKernelGGL((k64_argmax_bwd_both<PROD>), dim3((unsigned)total), dim3(64), 0, (hipStream_t)stream, a, b, idx,
                     g, grad_a, grad_b, M, K, N, row_tiles, kc_a, ps_a, col_tiles, kc_b, ps_b);
  return launch_status();
}

// The factored matrix-core kernels take problems big enough for their tiles to pay and small
// enough for a whole row or column of maxima in LDS.
inline bool d64_mm_ok(int B, int M, int K, int N) {
  if (B <= 0 || M <= 0 || K <= 0 || N <= 0) return false;
  const long ti = (M + 63) / 64, tk = (K + 63) / 64, tn = (N + 63) / 64;
  return (long)M * K * N >= 16 * 16 * 16 && max(M, N) <= kDMaxAll && B * max(ti * tn, max(ti * tk, tk * tn)) < 0x7fffffffL;
}
template <int KIND, int T>
inline void launch_d64_mm_t(const double* a, const double* b, const double* out, const double* g, double* dst, int B,
                            int M, int K, int N, hipStream_t s) {
  const int I = KIND == kD64GradB ? K : M, J = KIND == kD64GradA ? K : N;
  const int ti = (I + T - 1) / T, tj = (J + T - 1) / T;
  hipLaunchKernelGGL((k64_log_mm<KIND, T>), dim3((unsigned)((long)B * ti * tj)), dim3(4 * T),
                     d64_mm_lds(KIND, T, M, N), s, a, b, out, g, dst, M, K, N, ti, tj);
}
// 128 x 128 tiles (eight waves) where the result is wider than one 64 x 64 tile in both directions
// and the tile's LDS stays within the default 64 KB: half the exponentials per product, and an
// item of 128 x 128 takes its maxima and reads its operands once instead of four times.
template <int KIND>
inline void launch_d64_mm(const double* a, const double* b, const double* out, const double* g, double* dst, int B,
                          int M, int K, int N, hipStream_t s) {
  const int I = KIND == kD64GradB ? K : M, J = KIND == kD64GradA ? K : N;
  if (I > 64 && J > 64 && d64_mm_lds(KIND, 128, M, N) <= 64 * 1024)
    launch_d64_mm_t<KIND, 128>(a, b, out, g, dst, B, M, K, N, s);
  else
    launch_d64_mm_t<KIND, 64>(a, b, out, g, dst, B, M, K, N, s);
}
}  // namespace
}  // namespace GENBMM_NS

extern "C" {

int genbmm_logbmm_fwd_f64(const double* a, const double* b, double* out, int B, int M, int K, int N,
                          void* stream) {
  using namespace GENBMM_NS;
  if (d64_mm_ok(B, M, K, N)) {
    if (int e = check_dense_dims(B, M, K, N)) return e;
    if (!a || !b || !out) return GENBMM_E_NULLPTR;
    launch_d64_mm<kD64Fwd>(a, b, nullptr, nullptr, out, B, M, K, N, (hipStream_t)stream);
    return launch_status();
  }
  return run_fwd64<kLog>(a, b, out, nullptr, 0, 0, B, M, K, N, stream);
}

int genbmm_maxbmm_fwd_f64(const double* a, const double* b, double* out, int32_t* idx, int B, int M,
                          int K, int N, void* stream) {
  return GENBMM_NS::run_max_fwd64<false>(a, b, out, idx, B, M, K, N, stream);
}

int genbmm_prodmaxbmm_fwd_f64(const double* a, const double* b, double* out, int32_t* idx, int B,
                              int M, int K, int N, void* stream) {
  return GENBMM_NS::run_max_fwd64<true>(a, b, out, idx, B, M, K, N, stream);
}

int genbmm_samplebmm_fwd_f64(const double* a, const double* b, double* out, int32_t* idx,
                             uint64_t seed, uint64_t offset, int B, int M, int K, int N,
                             void* stream) {
  return GENBMM_NS::run_fwd64<GENBMM_NS::kSample>(a, b, out, idx, seed, offset, B, M, K, N, stream);
}

int genbmm_logbmm_bwd_f64(const double* a, const double* b, const double* out, const double* g,
                          double* grad_a, double* grad_b, int B, int M, int K, int N,
                          void* stream) {
  using namespace GENBMM_NS;
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(g, mn) ||
      missing(grad_a, mk) || missing(grad_b, kn))
    return GENBMM_E_NULLPTR;
  hipStream_t s = (hipStream_t)stream;
  if (d64_mm_ok(B, M, K, N)) {
    const size_t lds = max(d64_mm_lds(kD64GradA, 128, M, N), d64_mm_lds(kD64GradB, 128, M, N));
    if (max(max(M, K), N) <= 128 && min(min(M, K), N) > 64 && lds <= 64 * 1024) {  // one tile per item and gradient
      hipLaunchKernelGGL(k64_log_mm_both<128>, dim3((unsigned)((B + 7) / 8 * 16)), dim3(512), lds, s, a, b, out, g,
                         grad_a, grad_b, B, M, K, N);
      return launch_status();
    }
    launch_d64_mm<kD64GradA>(a, b, out, g, grad_a, B, M, K, N, s);
    launch_d64_mm<kD64GradB>(a, b, out, g, grad_b, B, M, K, N, s);
    return launch_status();
  }
  const int64_t rows = (int64_t)B * M;
  if (mk > 0) {
    if ((rows + 3) / 4 > 0x7fffffffLL) return GENBMM_E_SHAPE;
    hipLaunchKernelGGL(k64_log_bwd_a, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, a, b, out, g,
                       grad_a, M, K, N, (long)rows);
  }
  if (kn > 0)
    hipLaunchKernelGGL(k64_log_bwd_b, blocks_for(kn), dim3(256), 0, s, a, b, out, g, grad_b, M, K, N,
                       (long)kn);
  return launch_status();
}

int genbmm_logbmm_bwdbwd_f64(const double* a, const double* b, const double* out, const double* g,
                             const double* u_a, const double* u_b, double* grad_a, double* grad_b,
                             double* grad_g, int B, int M, int K, int N, void* stream) {
  using namespace GENBMM_NS;
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(g, mn) ||
      missing(grad_a, mk) || missing(grad_b, kn) || missing(grad_g, mn) ||
      (missing(u_a, mk) && missing(u_b, kn)))
    return GENBMM_E_NULLPTR;
  BB64 p{a, b, out, g, u_a, u_b, grad_a, grad_b, grad_g, M, K, N};
  hipStream_t s = (hipStream_t)stream;
  if (mn > 0) hipLaunchKernelGGL(k64_bb_t, blocks_for(mn), dim3(256), 0, s, p, (long)mn);
  if (mk > 0) hipLaunchKernelGGL(k64_bb_a, blocks_for(mk), dim3(256), 0, s, p, (long)mk);
  if (kn > 0) hipLaunchKernelGGL(k64_bb_b, blocks_for(kn), dim3(256), 0, s, p, (long)kn);
  return launch_status();
}

int genbmm_argmax_bwd_f64(const int32_t* idx, const double* g, double* grad_a, double* grad_b, int B,
                          int M, int K, int N, void* stream) {
  return GENBMM_NS::run_argmax_bwd64<false>(nullptr, nullptr, idx, g, grad_a, grad_b, B, M, K, N,
                                         stream);
}

int genbmm_prodmax_bwd_f64(const double* a, const double* b, const int32_t* idx, const double* g,
                           double* grad_a, double* grad_b, int B, int M, int K, int N,
                           void* stream) {
  return GENBMM_NS::run_argmax_bwd64<true>(a, b, idx, g, grad_a, grad_b, B, M, K, N, stream);
}

int genbmm_banded_fwd_f64(const double* a, int a_lu, int a_ld, const double* b, int b_lu, int b_ld,
                          double* out, int32_t* idx, int B, int n, int mode, void* stream) {
  using namespace GENBMM_NS;
  if (mode != GENBMM_BAND_LOG && mode != GENBMM_BAND_MAX && mode != GENBMM_BAND_MUL)
    return GENBMM_E_MODE;
  BandArgsT<double> p{};
  if (int e = fill_band(p, a_lu, a_ld, b_lu, b_ld, B, n)) return e;
  const long total = (long)B * n * p.Wo;
  if (total == 0) return GENBMM_OK;
  if (!a || !b || !out || (mode == GENBMM_BAND_MAX && !idx)) return GENBMM_E_NULLPTR;
  p.a = a; p.b = b; p.o0 = out; p.oidx = idx;
  hipStream_t s = (hipStream_t)stream;
  if (mode == GENBMM_BAND_LOG)
    hipLaunchKernelGGL((k_band_fwd<GENBMM_BAND_LOG, double>), blocks_for(total), dim3(256), 0, s, p, total);
  else if (mode == GENBMM_BAND_MAX)
    hipLaunchKernelGGL((k_band_fwd<GENBMM_BAND_MAX, double>), blocks_for(total), dim3(256), 0, s, p, total);
  else
    hipLaunchKernelGGL((k_band_fwd<GENBMM_BAND_MUL, double>), blocks_for(total), dim3(256), 0, s, p, total);
  return launch_status();
}

int genbmm_banded_sample_fwd_f64(const double* a, int a_lu, int a_ld, const double* b, int b_lu, int b_ld,
                                 double* out, int32_t* idx, uint64_t seed, uint64_t offset, int B, int n,
                                 void* stream) {
  using namespace GENBMM_NS;
  BandArgsT<double> p{};
  if (int e = fill_band(p, a_lu, a_ld, b_lu, b_ld, B, n)) return e;
  const long total = (long)B * n * p.Wo;
  if (total == 0) return GENBMM_OK;
  if (!a || !b || !out || !idx) return GENBMM_E_NULLPTR;
  p.a = a; p.b = b; p.o0 = out; p.oidx = idx;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL((k_band_fwd<GENBMM_BAND_LOG, double>), blocks_for(total), dim3(256), 0, s, p, total);
  hipLaunchKernelGGL(k_band_sample_cells<double>, blocks_for(total), dim3(256), 0, s, p, total, seed, offset);
  return launch_status();
}

int genbmm_banded_bwd_f64(const double* a, int a_lu, int a_ld, const double* b, int b_lu, int b_ld,
                          const double* out, const int32_t* idx, const double* g, double* grad_a,
                          double* grad_b, int B, int n, int mode, void* stream) {
  using namespace GENBMM_NS;
  if (mode == GENBMM_BAND_SAMPLE) mode = GENBMM_BAND_MAX;  // a drawn index scatters like an arg-max
  if (mode != GENBMM_BAND_LOG && mode != GENBMM_BAND_MAX && mode != GENBMM_BAND_MUL)
    return GENBMM_E_MODE;
  BandArgsT<double> p{};
  if (int e = fill_band(p, a_lu, a_ld, b_lu, b_ld, B, n)) return e;
  if ((int64_t)B * n == 0) return GENBMM_OK;
  if (!a || !b || !g || !grad_a || !grad_b || (mode == GENBMM_BAND_LOG && !out) ||
      (mode == GENBMM_BAND_MAX && !idx))
    return GENBMM_E_NULLPTR;
  p.a = a; p.b = b; p.out = out; p.idx = idx; p.g = g; p.o0 = grad_a; p.o1 = grad_b;
  const long ta = (long)B * n * p.Wa, tb = (long)B * n * p.Wb;
  hipStream_t s = (hipStream_t)stream;
  if (mode == GENBMM_BAND_LOG) {
    hipLaunchKernelGGL((k_band_bwd_a<GENBMM_BAND_LOG, double>), blocks_for(ta), dim3(256), 0, s, p, ta);
    hipLaunchKernelGGL((k_band_bwd_b<GENBMM_BAND_LOG, double>), blocks_for(tb), dim3(256), 0, s, p, tb);
  } else if (mode == GENBMM_BAND_MAX) {
    hipLaunchKernelGGL((k_band_bwd_a<GENBMM_BAND_MAX, double>), blocks_for(ta), dim3(256), 0, s, p, ta);
    hipLaunchKernelGGL((k_band_bwd_b<GENBMM_BAND_MAX, double>), blocks_for(tb), dim3(256), 0, s, p, tb);
  } else {
    hipLaunchKernelGGL((k_band_bwd_a<GENBMM_BAND_MUL, double>), blocks_for(ta), dim3(256), 0, s, p, ta);
    hipLaunchKernelGGL((k_band_bwd_b<GENBMM_BAND_MUL, double>), blocks_for(tb), dim3(256), 0, s, p, tb);
  }
  return launch_status();
}

int genbmm_banded_bwdbwd_f64(const double* a, int a_lu, int a_ld, const double* b, int b_lu,
                             int b_ld, const double* out, const double* g, const double* u_a,
                             const double* u_b, double* grad_a, double* grad_b, double* grad_g,
                             int B, int n, void* stream) {
  using namespace GENBMM_NS;
  BandArgsT<double> p{};
  if (int e = fill_band(p, a_lu, a_ld, b_lu, b_ld, B, n)) return e;
  if ((int64_t)B * n == 0) return GENBMM_OK;
  if (!a || !b || !out || !g || !grad_a || !grad_b || !grad_g || (!u_a && !u_b))
    return GENBMM_E_NULLPTR;
  p.a = a; p.b = b; p.out = out; p.g = g; p.ua = u_a; p.ub = u_b;
  p.o0 = grad_a; p.o1 = grad_b; p.o2 = grad_g;
  const long ta = (long)B * n * p.Wa, tb = (long)B * n * p.Wb, to = (long)B * n * p.Wo;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(k_band_bb_t<double>, blocks_for(to), dim3(256), 0, s, p, grad_g, to);
  hipLaunchKernelGGL(k_band_bb_a<double>, blocks_for(ta), dim3(256), 0, s, p, grad_g, ta);
  hipLaunchKernelGGL(k_band_bb_b<double>, blocks_for(tb), dim3(256), 0, s, p, grad_g, tb);
  return launch_status();
}

}  // extern "C"
