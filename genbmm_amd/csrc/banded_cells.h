// Band-product argument block and the per-cell routines: one output element
// computed straight from global memory, in the reference's loop order.  They
// are the whole kernel for max mode and for bands too wide for the strip
// kernels, and the exact recompute of single cells inside the strip kernels.
#pragma once

#include "common.h"

namespace GENBMM_NS {

// T: element type of the operands and results (float; double for the fp64 entry
// points, which run these per-cell kernels only).
template <class T>
struct BandArgsT {
  const T* a;
  const T* b;
  const T* out;
  const T* g;
  const T* ua;
  const T* ub;
  const int32_t* idx;
  T* o0;          // out        | grad_a
  T* o1;          // -          | grad_b
  T* o2;          // -          | grad_g
  int32_t* oidx;  // forward argmax
  // log product with a workspace: EA = exp(a - alpha), EB = exp(b - beta) with the
  // row maxima alpha, beta (over cells inside the matrix), and R = 1/S per output
  // cell (-1: the cell was computed exactly, S is not usable)
  float* ws_ea;
  float* ws_eb;
  float* ws_al;
  float* ws_be;
  float* ws_r;
  float* ws_h;    // backward scratch: g * R per output cell (NaN where R is not usable)
  int n, a_lu, Wa, b_lu, Wb, r_lu, Wo;
};
using BandArgs = BandArgsT<elem_t>;  // the caller's tensors; workspaces are float whatever the element type

// The type a cell is computed in: double for double tensors, float for float, binary16 and
// bfloat16 ones (widened by the load, rounded once by the store).
template <class T> struct band_acc { typedef float type; };
template <> struct band_acc<double> { typedef double type; };
template <class T> using band_acc_t = typename band_acc<T>::type;
// result -> element: one rounding to nearest even for the half types
template <class T, class A>
__device__ __forceinline__ T band_store(A x) {
  if constexpr (sizeof(T) == 2) return (T)settled((float)x);
  else return (T)x;
}

// exp of a difference and fused multiply-add per element type: float takes the
// hardware base-2 exponential, double the library routine.
__device__ __forceinline__ float sr_exp(float x) { return fast_exp(x); }
__device__ __forceinline__ double sr_exp(double x) { return exp(x); }
__device__ __forceinline__ float sr_fma(float x, float y, float z) { return __builtin_fmaf(x, y, z); }
__device__ __forceinline__ double sr_fma(double x, double y, double z) { return __builtin_fma(x, y, z); }

__device__ __forceinline__ int imax3(int a, int b, int c) { return max(a, max(b, c)); }
__device__ __forceinline__ int imin3(int a, int b, int c) { return min(a, min(b, c)); }

// Valid k range [klo, khi] of output cell (i, j); needs 0 <= o < n.
template <class T>
__device__ __forceinline__ void k_range(const BandArgsT<T>& p, int i, int j, int& klo, int& khi) {
  klo = imax3(0, j - (p.Wb - 1), p.a_lu - i);
  khi = imin3(p.Wa - 1, j, p.n - 1 + p.a_lu - i);
}

// ------------------------------------------------------------------ forward
// Reference banded_cuda_forward_kernel_mul (banded_cuda_kernel.cu:13-100).
// One output cell e = (bi*Wo + j), bi = batch*n + i.
template <int MODE, class T>
__device__ __forceinline__ void band_fwd_cell(const BandArgsT<T>& p, long bi, int i, int j) {
  typedef band_acc_t<T> A;
  const long e = bi * p.Wo + j;
  const int o = i + j - p.r_lu;
  if (o < 0 || o >= p.n) {  // outside the matrix: the reference leaves its zero fill
    p.o0[e] = (T)0;
    if (MODE == GENBMM_BAND_MAX) p.oidx[e] = 0;
    return;
  }
  int klo, khi;
  k_range(p, i, j, klo, khi);
  const T* ar = p.a + bi * p.Wa;
  const T* br = p.b + (bi + (o - i)) * p.Wb + (p.Wb - 1 - j);  // br[k] = b[o][k2(k)]
  if (MODE == GENBMM_BAND_MUL) {
    A v = 0;
    for (int k = klo; k <= khi; ++k) v = sr_fma((A)ar[k], (A)br[k], v);
    p.o0[e] = band_store<T>(v);
  } else if (MODE == GENBMM_BAND_MAX) {
    A m = kFloor;
    int ind = -1;
    for (int k = klo; k <= khi; ++k) {
      const A v = (A)ar[k] + (A)br[k];
      if (v > m) {
        m = v;
        ind = k;
      }
    }
    p.o0[e] = band_store<T>(m);
    p.oidx[e] = ind;
  } else if constexpr (sizeof(A) == sizeof(float)) {
    float m = kFloor;
    for (int k = klo; k <= khi; ++k) m = fmaxf(m, (float)ar[k] + (float)br[k]);
    const float nm = -m * kLog2e;
    float s = 0.f;
    for (int k = klo; k <= khi; ++k) s += fast_exp2(__builtin_fmaf((float)ar[k] + (float)br[k], kLog2e, nm));
    p.o0[e] = band_store<T>(logf(s) + m);
  } else {
    A m = kFloor;
    for (int k = klo; k <= khi; ++k) m = fmax(m, ar[k] + br[k]);
    A s = 0;
    for (int k = klo; k <= khi; ++k) s += exp(ar[k] + br[k] - m);
    p.o0[e] = log(s) + m;
  }
}

// ----------------------------------------------------------------- backward
// d out[i,j] / d a[i,k]: MUL b[o,k2]; LOG exp(a[i,k]+b[o,k2]-out[i,j]);
// MAX [k == idx[i,j]].  grad_a[i,k] sums over j ascending (reference
// banded_cuda_backward_kernel_mul, banded_cuda_kernel.cu:104-152).
template <int MODE, class T>
__device__ __forceinline__ void band_bwd_a_cell(const BandArgsT<T>& p, long bi, int i, int k) {
  typedef band_acc_t<T> A;
  const long e = bi * p.Wa + k;
  const int pos = i + k - p.a_lu;
  A acc = 0;
  if (pos >= 0 && pos < p.n) {
    const int jlo = imax3(k, p.r_lu - i, 0);
    const int jhi = imin3(k + p.Wb - 1, p.n - 1 + p.r_lu - i, p.Wo - 1);
    const T* gr = p.g + bi * p.Wo;
    // b[o][k2] = bw[j * (Wb - 1)] with o = i + j - r_lu, k2 = k - j + Wb - 1
    const T* bw = p.b + (bi - p.r_lu) * p.Wb + k + p.Wb - 1;
    if (MODE == GENBMM_BAND_MUL) {
      for (int j = jlo; j <= jhi; ++j) acc = sr_fma((A)bw[(long)j * (p.Wb - 1)], (A)gr[j], acc);
    } else if (MODE == GENBMM_BAND_MAX) {
      const int32_t* ir = p.idx + bi * p.Wo;
      for (int j = jlo; j <= jhi; ++j) acc += (ir[j] == k) ? (A)gr[j] : A(0);
    } else {
      const A av = p.a[e];
      const T* orow = p.out + bi * p.Wo;
      for (int j = jlo; j <= jhi; ++j) {
        const A w = sr_exp(av + (A)bw[(long)j * (p.Wb - 1)] - (A)orow[j]);
        acc = sr_fma(w, (A)gr[j], acc);
      }
    }
  }
  p.o0[e] = band_store<T>(acc);
}

// grad_b[o,k2] sums, in ascending i, over the cells (i, j = o - i + r_lu) that
// read b[o,k2], with k = k2 + j - (Wb - 1).  The reference gets the same
// numbers by transposing g / out in band form on the host and calling the
// kernel above with the operands swapped (sparse.py:436-446, 523-545, 625-635).
template <int MODE, class T>
__device__ __forceinline__ void band_bwd_b_cell(const BandArgsT<T>& p, long bo, int o, int k2) {
  typedef band_acc_t<T> A;
  const long e = bo * p.Wb + k2;
  const int prow = o + k2 - p.b_lu;
  A acc = 0;
  if (prow >= 0 && prow < p.n) {
    const int jhi_k = p.Wb - 1 - k2 + p.Wa - 1;  // j with k = Wa-1
    const int jlo_k = p.Wb - 1 - k2;             // j with k = 0
    const int ilo = imax3(0, o + p.r_lu - min(jhi_k, p.Wo - 1), o + p.r_lu - (p.Wo - 1));
    const int ihi = imin3(p.n - 1, o + p.r_lu - max(jlo_k, 0), o + p.r_lu);
    const long base = bo - o;  // batch*n
    const A bv = p.b[e];
    for (int i = ilo; i <= ihi; ++i) {
      const int j = o - i + p.r_lu;
      const int k = k2 + j - (p.Wb - 1);
      const long gi = (base + i) * p.Wo + j;
      if (MODE == GENBMM_BAND_MUL) {
        acc = sr_fma((A)p.a[(base + i) * p.Wa + k], (A)p.g[gi], acc);
      } else if (MODE == GENBMM_BAND_MAX) {
        acc += (p.idx[gi] == k) ? (A)p.g[gi] : A(0);
      } else {
        const A w = sr_exp((A)p.a[(base + i) * p.Wa + k] + bv - (A)p.out[gi]);
        acc = sr_fma(w, (A)p.g[gi], acc);
      }
    }
  }
  p.o1[e] = band_store<T>(acc);
}

// ------------------------------------------------ one lane per cell kernels
template <int MODE, class T>
__global__ __launch_bounds__(256) void k_band_fwd(const BandArgsT<T> p, long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const long bi = e / p.Wo;  // batch*n + i
  band_fwd_cell<MODE>(p, bi, (int)(bi % p.n), (int)(e - bi * p.Wo));
}

template <int MODE, class T>
__global__ __launch_bounds__(256) void k_band_bwd_a(const BandArgsT<T> p, long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const long bi = e / p.Wa;
  band_bwd_a_cell<MODE>(p, bi, (int)(bi % p.n), (int)(e - bi * p.Wa));
}

template <int MODE, class T>
__global__ __launch_bounds__(256) void k_band_bwd_b(const BandArgsT<T> p, long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const long bo = e / p.Wb;
  band_bwd_b_cell<MODE>(p, bo, (int)(bo % p.n), (int)(e - bo * p.Wb));
}

// ------------------------------------------------------------------ sample
// The banded sample product (no counterpart among the reference's band modes): the dense
// sampling rule (sample_cuda_forward_kernel, matmul_cuda_kernel.cu:107-118) on the terms of
// a band cell in ascending k.
// The exact walk of one cell inside the matrix, u its uniform; returns the index.
template <class T>
__device__ __forceinline__ int band_sample_cell(const BandArgsT<T>& p, long bi, int i, int j, float u) {
  const int o = i + j - p.r_lu;
  int klo, khi;
  k_range(p, i, j, klo, khi);
  const T* ar = p.a + bi * p.Wa;
  const T* br = p.b + (bi + (o - i)) * p.Wb + (p.Wb - 1 - j);
  if constexpr (sizeof(T) == sizeof(double)) {
    double m = kFloor;
    for (int k = klo; k <= khi; ++k) m = fmax(m, (double)ar[k] + (double)br[k]);
    double s = 0;
    for (int k = klo; k <= khi; ++k) s += exp((double)ar[k] + (double)br[k] - m);
    const double t = (double)u * s;
    double tot = 0;
    int last = klo;
    for (int k = klo; k <= khi; ++k) {
      const double pr = exp((double)ar[k] + (double)br[k] - m);
      if (tot + pr > t) return k;  // (total < t holds until then, except on an exact tie, which the next term takes)
      tot += pr;
      if (pr > 0) last = k;
    }
    return u > 0.f ? last : klo;
  } else {
    float m = kFloor;
    for (int k = klo; k <= khi; ++k) m = fmaxf(m, (float)ar[k] + (float)br[k]);
    const float nm = -m * kLog2e;
    float s = 0.f;
    for (int k = klo; k <= khi; ++k) s += fast_exp2(__builtin_fmaf((float)ar[k] + (float)br[k], kLog2e, nm));
    const float t = u * s;
    float tot = 0.f;
    int last = klo;
    for (int k = klo; k <= khi; ++k) {
      const float pr = fast_exp2(__builtin_fmaf((float)ar[k] + (float)br[k], kLog2e, nm));
      if (tot + pr > t) return k;  // (total < t holds until then, except on an exact tie, which the next term takes)
      tot += pr;
      if (pr > 0.f) last = k;
    }
    // ran out by rounding: the last term that had mass (r = 0 brackets nothing: first term)
    return u > 0.f ? last : klo;
  }
}

// One lane per cell: the exact walk everywhere.
template <class T>
__global__ __launch_bounds__(256) void k_band_sample_cells(const BandArgsT<T> p, long total, uint64_t seed,
                                                           uint64_t offset) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const long bi = e / p.Wo;
  const int i = (int)(bi % p.n), j = (int)(e - bi * p.Wo), o = i + j - p.r_lu;
  p.oidx[e] = (o < 0 || o >= p.n) ? 0 : band_sample_cell(p, bi, i, j, philox_uniform((uint64_t)e, seed, offset));
}

// ------------------------------------------------------ log second order
// p = exp(a[i,k] + b[o,k2] - out[i,j]),  w = u_a[i,k] + u_b[o,k2]:
//   t[i,j]       = sum_k p*w                        (gradient w.r.t. g)
//   grad_a[i,k]  = sum_j g[i,j]*p*(w - t[i,j])
//   grad_b[o,k2] = sum_i g[i,j]*p*(w - t[i,j])
// With u_b = 0 these equal the reference's banded_cuda_backbackward_kernel_A/
// _B/_C (banded_cuda_kernel.cu:154-350), whose inner loop sum_m (delta*s -
// s*s2)*u[m] is s*(u[k] - t).
// `tt`: t per output cell in the accumulation type (a float buffer of the caller's for
// the half element types, whose grad_g output holds t rounded; else grad_g itself).
template <class T>
__global__ __launch_bounds__(256) void k_band_bb_t(const BandArgsT<T> p, band_acc_t<T>* __restrict__ tt, long total) {
  typedef band_acc_t<T> A;
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int j = (int)(e % p.Wo);
  const long bi = e / p.Wo;
  const int i = (int)(bi % p.n);
  const int o = i + j - p.r_lu;
  A t = 0;
  if (o >= 0 && o < p.n) {
    int klo, khi;
    k_range(p, i, j, klo, khi);
    const long boff = (bi + (o - i)) * p.Wb + (p.Wb - 1 - j);
    const A ov = p.out[e];
    for (int k = klo; k <= khi; ++k) {
      const A pr = sr_exp((A)p.a[bi * p.Wa + k] + (A)p.b[boff + k] - ov);
      const A w = (p.ua ? (A)p.ua[bi * p.Wa + k] : A(0)) + (p.ub ? (A)p.ub[boff + k] : A(0));
      t = sr_fma(pr, w, t);
    }
  }
  tt[e] = t;
  if constexpr (sizeof(T) != sizeof(A)) p.o2[e] = band_store<T>(t);
}

template <class T>
__global__ __launch_bounds__(256) void k_band_bb_a(const BandArgsT<T> p, const band_acc_t<T>* __restrict__ tt,
                                                   long total) {
  typedef band_acc_t<T> A;
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int k = (int)(e % p.Wa);
  const long bi = e / p.Wa;
  const int i = (int)(bi % p.n);
  const int pos = i + k - p.a_lu;
  A acc = 0;
  if (pos >= 0 && pos < p.n) {
    const int jlo = imax3(k, p.r_lu - i, 0);
    const int jhi = imin3(k + p.Wb - 1, p.n - 1 + p.r_lu - i, p.Wo - 1);
    const long bw = (bi - p.r_lu) * p.Wb + k + p.Wb - 1;
    const A av = p.a[e];
    const A uav = p.ua ? (A)p.ua[e] : A(0);
    for (int j = jlo; j <= jhi; ++j) {
      const long bj = bw + (long)j * (p.Wb - 1);
      const long gi = bi * p.Wo + j;
      const A pr = sr_exp(av + (A)p.b[bj] - (A)p.out[gi]);
      const A w = uav + (p.ub ? (A)p.ub[bj] : A(0)) - tt[gi];
      acc = sr_fma((A)p.g[gi] * pr, w, acc);
    }
  }
  p.o0[e] = band_store<T>(acc);
}

template <class T>
__global__ __launch_bounds__(256) void k_band_bb_b(const BandArgsT<T> p, const band_acc_t<T>* __restrict__ tt,
                                                   long total) {
  typedef band_acc_t<T> A;
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int k2 = (int)(e % p.Wb);
  const long bo = e / p.Wb;
  const int o = (int)(bo % p.n);
  const int prow = o + k2 - p.b_lu;
  A acc = 0;
  if (prow >= 0 && prow < p.n) {
    const int jhi_k = p.Wb - 1 - k2 + p.Wa - 1;
    const int jlo_k = p.Wb - 1 - k2;
    const int ilo = imax3(0, o + p.r_lu - min(jhi_k, p.Wo - 1), o + p.r_lu - (p.Wo - 1));
    const int ihi = imin3(p.n - 1, o + p.r_lu - max(jlo_k, 0), o + p.r_lu);
    const long base = bo - o;
    const A bv = p.b[e];
    const A ubv = p.ub ? (A)p.ub[e] : A(0);
    for (int i = ilo; i <= ihi; ++i) {
      const int j = o - i + p.r_lu;
      const int k = k2 + j - (p.Wb - 1);
      const long gi = (base + i) * p.Wo + j;
      const long ai = (base + i) * p.Wa + k;
      const A pr = sr_exp((A)p.a[ai] + bv - (A)p.out[gi]);
      const A w = (p.ua ? (A)p.ua[ai] : A(0)) + ubv - tt[gi];
      acc = sr_fma((A)p.g[gi] * pr, w, acc);
    }
  }
  p.o1[e] = band_store<T>(acc);
}

// ------------------------------------------------------------------- host
template <class T>
inline int fill_band(BandArgsT<T>& p, int a_lu, int a_ld, int b_lu, int b_ld, int B, int n) {
  if (a_lu < 0 || a_ld < 0 || b_lu < 0 || b_ld < 0) return GENBMM_E_BAND;
  if (B < 0 || n < 0) return GENBMM_E_SHAPE;
  const int64_t Wa = (int64_t)a_lu + a_ld + 1, Wb = (int64_t)b_lu + b_ld + 1;
  const int64_t Wo = Wa + Wb - 1;
  // 2^37 cells: beyond any device buffer, and one-lane-per-cell grids (cells / 256) stay within
  // 32 bits; the strip and tile-row kernels launch at most two workgroups per 16 rows and
  // segment of 8 result diagonals - a grid beyond 2^31 - 1 workgroups would wrap silently
  if (Wo > 0x3fffffff || (int64_t)B * n * Wo > ((int64_t)1 << 37)) return GENBMM_E_SHAPE;
  if ((int64_t)B * ((n + 15) / 16) * ((Wo + 7) / 8) > ((int64_t)1 << 30)) return GENBMM_E_SHAPE;
  p.n = n; p.a_lu = a_lu; p.Wa = (int)Wa; p.b_lu = b_lu; p.Wb = (int)Wb;
  p.r_lu = a_lu + b_ld; p.Wo = (int)Wo;
  return GENBMM_OK;
}

inline dim3 blocks_for(long total) { return dim3((unsigned)((total + 255) / 256)); }

}  // namespace GENBMM_NS
