// Banded sample product: out = banded log-sum-exp, idx[i,j] = a term k of cell (i, j) drawn
// with probability exp(a[i,k] + b[o,k2] - out[i,j]) (index into a's band, as the max product
// stores its arg-max).  The reference's band kernel has no such mode
// (banded_cuda_kernel.cu:42, 65, 76 handle 0, 1 and 3); the rule is its dense one
// (sample_cuda_forward_kernel, matmul_cuda_kernel.cu:107-118) on a band cell's terms in
// ascending k: the first term with total < r && total + p > r, r the cell's uniform; a cell
// whose walk never brackets r keeps its first term (the dense kernel keeps index 0, its first
// term); cells outside the matrix keep index 0.  r of cell e = (batch * n + i) * Wo + j is
// the Philox4x32-10 uniform of that cell index, as in the dense product.
//
// On the log product's workspace (EA = exp(a - rowmax), EB, 1/S per cell) the walk needs no
// exponential: with the target t = r * S the index is the number of prefix sums of EA * EB
// that do not exceed t.  k_band_sample_targets writes t into the index tensor (as float
// bits; -1 where 1/S is not usable), k_band_sample_fwd - the whole-strip walk of the max
// product on the prepared operands, which hold zeros outside the matrix - replaces it by the
// index.  Cells without a usable 1/S, and bands the strip kernel does not take, walk exactly
// (band_sample_cell: running maximum, sum, then the rule on exp(v - max) against r * sum).
#pragma once

#include "banded_max.h"

namespace GENBMM_NS {

// Targets shrink by 2^-17 of themselves: the prefix sums here and the forward's S are added
// in different orders, and a uniform within rounding of 1 must still land on a term.
constexpr float kBandSampleShrink = 1.f - 1.f / 131072.f;

// idx[e] <- bits of r(e) / R[e], shrunk; -1.0f where R is not usable (the forward computed the
// cell exactly), -2.0f outside the matrix.  Four cells per lane, one Philox block each.
__global__ __launch_bounds__(256) void k_band_sample_targets(const float* __restrict__ r, int32_t* __restrict__ idx,
                                                             long cells, uint64_t seed, uint64_t offset) {
  const long q = (long)blockIdx.x * 256 + threadIdx.x;
  const long e0 = 4 * q;
  if (e0 >= cells) return;
  const Philox4 x = philox_block((uint64_t)q, seed, offset);
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    if (e0 + t < cells) {
      const float rv = r[e0 + t];
      const float u = philox_scale(x.x[t]);
      const float tg = rv > 0.f ? u * __builtin_amdgcn_rcpf(rv) * kBandSampleShrink : (rv < 0.f ? -1.f : -2.f);
      idx[e0 + t] = __float_as_int(tg);
    }
  }
}

// The whole-strip walk (k_band_max_fwd's staging and cell ownership) on EA and EB.
template <class T>
__global__ __launch_bounds__(256, 2) void k_band_sample_fwd(const BandArgsT<T> p, int strips, const MaxDims d,
                                                            long cells_a, long cells_b, int nseg, int Wseg,
                                                            uint64_t seed, uint64_t offset) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int wg = xcd_strip_id();
  const int seg = wg % nseg;
  wg /= nseg;
  const int batch = wg / strips, x0 = (wg - batch * strips) * kMaxRows;
  const int n = p.n, Wa = p.Wa, Wb = p.Wb, Wo = p.Wo, r_lu = p.r_lu;
  const int j_lo = seg * Wseg, Ws = min(Wseg, Wo - j_lo);
  const long bn = (long)batch * n;
  float* PL = smem + kMmSlack;
  float* QL = smem + d.q_off;

  // ---- staging: EA rows of the strip, the EB rows its cells meet, zeros between the rows
  const int q0 = x0 - r_lu + j_lo;
  const int qr0 = max(q0, 0), qr1 = min(q0 + d.q_rows, n);
  const int pr1 = min(x0 + kMaxRows, n);
  MmFlat<14> sq;
  MmFlat<6> sp;
  sq.init(p.ws_eb, p.ws_eb + cells_b, (bn + qr0) * Wb, (qr1 - qr0) * Wb, Wb, d.qp);
  sq.load(p.ws_eb, p.ws_eb + cells_b, 0, tid);
  sp.init(p.ws_ea, p.ws_ea + cells_a, (bn + x0) * Wa, (pr1 - x0) * Wa, Wa, d.pp);
  sp.load(p.ws_ea, p.ws_ea + cells_a, 0, tid);
  sq.store(QL, 0, tid);
  for (int b = 1; sq.more(b); ++b) {
    sq.load(p.ws_eb, p.ws_eb + cells_b, b, tid);
    sq.store(QL, b, tid);
  }
  sp.store(PL, 0, tid);
  for (int b = 1; sp.more(b); ++b) {
    sp.load(p.ws_ea, p.ws_ea + cells_a, b, tid);
    sp.store(PL, b, tid);
  }
  {
    const int gap = d.qp - Wb, first = sq.origin() - (qr0 - q0) * d.qp;
    for (int e = tid; e < (d.q_rows + 1) * gap; e += 256) {
      const int r = e / gap, c = e - r * gap;
      const int at = first + (r - 1) * d.qp + Wb + c;
      if (at >= 0) QL[at] = 0.f;
    }
  }
  __syncthreads();
  const int pp = d.pp, qp = d.qp;
  const float* Pt = PL + sp.origin();
  const float* Qt = QL + sq.origin() - (qr0 - q0) * qp;

  // ---- walks
  const int x = x0 + lane;
  const bool interior = x0 >= max(p.a_lu, r_lu) && x0 + kMaxRows - 1 <= n - 1 - max(Wa - 1 - p.a_lu, Wo - 1 - r_lu);
  const float* ap = Pt + lane * pp;
  const int nblocks = (Ws + 7) >> 3;
  const int32_t* trow = p.oidx + (bn + min(x, n - 1)) * Wo;  // the targets of this lane's row
  int ind[5][8];
#pragma unroll
  for (int s = 0; s < 5; ++s) {
#pragma unroll
    for (int t = 0; t < 8; ++t) ind[s][t] = 0;
    const int jb = wave + 4 * s;
    if (jb < nblocks) {
      const int j0 = j_lo + 8 * jb;
      float tg[8], acc[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        tg[t] = __int_as_float(trow[min(j0 + t, Wo - 1)]);
        acc[t] = 0.f;
      }
      const float* bp = Qt + (lane + j0 - j_lo) * qp + (Wb - 1 - j0);
      const int dt = qp - 1;
      // the index is the number of prefix sums that do not exceed the target (they never decrease)
      auto fold = [&](int t, float av, float bv) __attribute__((always_inline)) {
        acc[t] = __builtin_fmaf(av, bv, acc[t]);
        ind[s][t] += acc[t] <= tg[t] ? 1 : 0;
      };
      if (interior) {
        const int klo = max(0, j0 - (Wb - 1)), khi = min(Wa - 1, j0 + 7);
        int k = klo;
        for (; k + 3 <= khi; k += 4) {
          float av[4], bv[4][8];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            av[u] = ap[k + u];
#pragma unroll
            for (int t = 0; t < 8; ++t) bv[u][t] = bp[t * dt + k + u];
          }
#pragma unroll
          for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int t = 0; t < 8; ++t) fold(t, av[u], bv[u][t]);
        }
        for (; k <= khi; ++k) {
          const float av = ap[k];
#pragma unroll
          for (int t = 0; t < 8; ++t) fold(t, av, bp[t * dt + k]);
        }
        // cells of the block start their count at the first k of the union
#pragma unroll
        for (int t = 0; t < 8; ++t) ind[s][t] += klo;
      } else if (x < n) {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          const int j = j0 + t, o = x + j - r_lu;
          if (j < j_lo + Ws && o >= 0 && o < n) {
            const int klo = max(max(0, j - (Wb - 1)), p.a_lu - x), khi = min(min(Wa - 1, j), n - 1 + p.a_lu - x);
            for (int k = klo; k <= khi; ++k) fold(t, ap[k], bp[t * dt + k]);
            ind[s][t] += klo;
          }
        }
      }
      // into the cell's own range of k (a target that no prefix exceeds, by rounding: the last
      // term); cells without a usable 1/S walk exactly; outside the matrix: 0
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int j = j0 + t, o = x + j - r_lu;
        int v = 0;
        if (x < n && j < j_lo + Ws && o >= 0 && o < n) {
          if (tg[t] >= 0.f) {
            const int klo = max(max(0, j - (Wb - 1)), p.a_lu - x), khi = min(min(Wa - 1, j), n - 1 + p.a_lu - x);
            v = min(max(ind[s][t], klo), khi);
          } else {
            const long e = (bn + x) * Wo + j;
            v = band_sample_cell(p, bn + x, x, j, philox_uniform((uint64_t)e, seed, offset));
          }
        }
        ind[s][t] = v;
      }
    }
  }
  __syncthreads();  // the operands are consumed: their place becomes the index tile

  int* Si = reinterpret_cast<int*>(smem);
#pragma unroll
  for (int s = 0; s < 5; ++s) {
    const int jb = wave + 4 * s;
    if (jb < nblocks) {
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int js = 8 * jb + t;
        if (js < Ws) Si[lane * Ws + js] = ind[s][t];
      }
    }
  }
  __syncthreads();
  const int rows = min(kMaxRows, n - x0), cells = rows * Ws;
  int32_t* ib = p.oidx + (bn + x0) * Wo + j_lo;
  typedef int mm_i4 __attribute__((ext_vector_type(4)));
  if (Ws == Wo && (cells & 3) == 0 && (reinterpret_cast<uintptr_t>(ib) & 15) == 0) {
    for (int e = 4 * tid; e < cells; e += 1024) *reinterpret_cast<mm_i4*>(ib + e) = *reinterpret_cast<const mm_i4*>(Si + e);
  } else {
    for (int e = tid; e < cells; e += 256) {
      const int r = e / Ws, c = e - r * Ws;
      ib[(long)r * Wo + c] = Si[e];
    }
  }
}

}  // namespace GENBMM_NS
