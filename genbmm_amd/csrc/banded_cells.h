// Band-product argument block and the per-cell routines: one output element
// computed straight from global memory, in the reference's loop order.  They
// are the whole kernel for max mode and for bands too wide for the strip
// kernels, and the exact recompute of single cells inside the strip kernels.
#pragma once

#include "common.h"

namespace genbmm {

struct BandArgs {
  const float* a;
  const float* b;
  const float* out;
  const float* g;
  const float* ua;
  const float* ub;
  const int32_t* idx;
  float* o0;      // out        | grad_a
  float* o1;      // -          | grad_b
  float* o2;      // -          | grad_g
  int32_t* oidx;  // forward argmax
  // log product with a workspace: EA = exp(a - alpha), EB = exp(b - beta) with the
  // row maxima alpha, beta (over cells inside the matrix), and R = 1/S per output
  // cell (-1: the cell was computed exactly, S is not usable)
  float* ws_ea;
  float* ws_eb;
  float* ws_al;
  float* ws_be;
  float* ws_r;
  int n, a_lu, Wa, b_lu, Wb, r_lu, Wo;
};

__device__ __forceinline__ int imax3(int a, int b, int c) { return max(a, max(b, c)); }
__device__ __forceinline__ int imin3(int a, int b, int c) { return min(a, min(b, c)); }

// Valid k range [klo, khi] of output cell (i, j); needs 0 <= o < n.
__device__ __forceinline__ void k_range(const BandArgs& p, int i, int j, int& klo, int& khi) {
  klo = imax3(0, j - (p.Wb - 1), p.a_lu - i);
  khi = imin3(p.Wa - 1, j, p.n - 1 + p.a_lu - i);
}

// ------------------------------------------------------------------ forward
// Reference banded_cuda_forward_kernel_mul (banded_cuda_kernel.cu:13-100).
// One output cell e = (bi*Wo + j), bi = batch*n + i.
template <int MODE>
__device__ __forceinline__ void band_fwd_cell(const BandArgs& p, long bi, int i, int j) {
  const long e = bi * p.Wo + j;
  const int o = i + j - p.r_lu;
  if (o < 0 || o >= p.n) {  // outside the matrix: the reference leaves its zero fill
    p.o0[e] = 0.f;
    if (MODE == GENBMM_BAND_MAX) p.oidx[e] = 0;
    return;
  }
  int klo, khi;
  k_range(p, i, j, klo, khi);
  const float* ar = p.a + bi * p.Wa;
  const float* br = p.b + (bi + (o - i)) * p.Wb + (p.Wb - 1 - j);  // br[k] = b[o][k2(k)]
  if (MODE == GENBMM_BAND_MUL) {
    float v = 0.f;
    for (int k = klo; k <= khi; ++k) v = __builtin_fmaf(ar[k], br[k], v);
    p.o0[e] = v;
  } else if (MODE == GENBMM_BAND_MAX) {
    float m = kFloor;
    int ind = -1;
    for (int k = klo; k <= khi; ++k) {
      const float v = ar[k] + br[k];
      if (v > m) {
        m = v;
        ind = k;
      }
    }
    p.o0[e] = m;
    p.oidx[e] = ind;
  } else {
    float m = kFloor;
    for (int k = klo; k <= khi; ++k) m = fmaxf(m, ar[k] + br[k]);
    const float nm = -m * kLog2e;
    float s = 0.f;
    for (int k = klo; k <= khi; ++k) s += fast_exp2(__builtin_fmaf(ar[k] + br[k], kLog2e, nm));
    p.o0[e] = logf(s) + m;
  }
}

// ----------------------------------------------------------------- backward
// d out[i,j] / d a[i,k]: MUL b[o,k2]; LOG exp(a[i,k]+b[o,k2]-out[i,j]);
// MAX [k == idx[i,j]].  grad_a[i,k] sums over j ascending (reference
// banded_cuda_backward_kernel_mul, banded_cuda_kernel.cu:104-152).
template <int MODE>
__device__ __forceinline__ void band_bwd_a_cell(const BandArgs& p, long bi, int i, int k) {
  const long e = bi * p.Wa + k;
  const int pos = i + k - p.a_lu;
  float acc = 0.f;
  if (pos >= 0 && pos < p.n) {
    const int jlo = imax3(k, p.r_lu - i, 0);
    const int jhi = imin3(k + p.Wb - 1, p.n - 1 + p.r_lu - i, p.Wo - 1);
    const float* gr = p.g + bi * p.Wo;
    // b[o][k2] = bw[j * (Wb - 1)] with o = i + j - r_lu, k2 = k - j + Wb - 1
    const float* bw = p.b + (bi - p.r_lu) * p.Wb + k + p.Wb - 1;
    if (MODE == GENBMM_BAND_MUL) {
      for (int j = jlo; j <= jhi; ++j) acc = __builtin_fmaf(bw[(long)j * (p.Wb - 1)], gr[j], acc);
    } else if (MODE == GENBMM_BAND_MAX) {
      const int32_t* ir = p.idx + bi * p.Wo;
      for (int j = jlo; j <= jhi; ++j) acc += (ir[j] == k) ? gr[j] : 0.f;
    } else {
      const float av = p.a[e];
      const float* orow = p.out + bi * p.Wo;
      for (int j = jlo; j <= jhi; ++j) {
        const float w = fast_exp(av + bw[(long)j * (p.Wb - 1)] - orow[j]);
        acc = __builtin_fmaf(w, gr[j], acc);
      }
    }
  }
  p.o0[e] = acc;
}

// grad_b[o,k2] sums, in ascending i, over the cells (i, j = o - i + r_lu) that
// read b[o,k2], with k = k2 + j - (Wb - 1).  The reference gets the same
// numbers by transposing g / out in band form on the host and calling the
// kernel above with the operands swapped (sparse.py:436-446, 523-545, 625-635).
template <int MODE>
__device__ __forceinline__ void band_bwd_b_cell(const BandArgs& p, long bo, int o, int k2) {
  const long e = bo * p.Wb + k2;
  const int prow = o + k2 - p.b_lu;
  float acc = 0.f;
  if (prow >= 0 && prow < p.n) {
    const int jhi_k = p.Wb - 1 - k2 + p.Wa - 1;  // j with k = Wa-1
    const int jlo_k = p.Wb - 1 - k2;             // j with k = 0
    const int ilo = imax3(0, o + p.r_lu - min(jhi_k, p.Wo - 1), o + p.r_lu - (p.Wo - 1));
    const int ihi = imin3(p.n - 1, o + p.r_lu - max(jlo_k, 0), o + p.r_lu);
    const long base = bo - o;  // batch*n
    const float bv = p.b[e];
    for (int i = ilo; i <= ihi; ++i) {
      const int j = o - i + p.r_lu;
      const int k = k2 + j - (p.Wb - 1);
      const long gi = (base + i) * p.Wo + j;
      if (MODE == GENBMM_BAND_MUL) {
        acc = __builtin_fmaf(p.a[(base + i) * p.Wa + k], p.g[gi], acc);
      } else if (MODE == GENBMM_BAND_MAX) {
        acc += (p.idx[gi] == k) ? p.g[gi] : 0.f;
      } else {
        const float w = fast_exp(p.a[(base + i) * p.Wa + k] + bv - p.out[gi]);
        acc = __builtin_fmaf(w, p.g[gi], acc);
      }
    }
  }
  p.o1[e] = acc;
}

}  // namespace genbmm
