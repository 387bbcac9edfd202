// Banded max-plus forward on whole strips: out[i,j] = max_k a[i,k] + b[o,k2] with its
// arg-max k (lowest k on ties, strict '>' from the reference's -1e9 floor, -1 if no k),
// o = i + j - lu_out, k2 = k - j + Wb - 1.
//
// A workgroup owns 64 rows i.  Their rows of a and the 64 + Wo - 1 rows of b that they
// meet are copied to LDS once, as they lie in memory (16-byte pieces, odd row strides: the
// 64 lanes of a wave are 64 consecutive rows and fall in different banks).  A lane owns
// one row; a wave walks blocks of 8 adjacent result diagonals j (blocks w, w + 4, ...
// - their sum lengths pair up, so the four waves get equal work), reading one value of
// its own row per k and 8 values of b on an anti-diagonal.  The 8 cells walk the union of
// their k ranges without predicates: the rows of b lie at least 7 cells apart in LDS, with
// -inf between them.  Strips that touch the matrix edge take a loop with the per-cell k
// range of the reference instead.  Values and indices go
// through LDS so that the strip's rows are written as one contiguous run.
//
// Compared with the chunked strip kernel (banded_strip.h) the sliding operand is staged
// once instead of once per 32 diagonals, and the result leaves in 16-byte stores.
//
// Wide results are cut into segments of Wseg <= 160 adjacent diagonals, one workgroup per strip
// and segment: a segment needs only the 64 + Wseg - 1 rows of b that its diagonals meet, so the
// tiles fit in LDS whatever the band width; its cells leave as one run of Wseg per row.
#pragma once

#include "banded_flat.h"

namespace GENBMM_NS {

constexpr int kMaxRows = 64;

struct MaxDims {
  int pp, qp, q_off, ops_floats, q_rows;
  size_t bytes;
};

// Wo: the diagonals one workgroup takes (the whole result or a segment of it)
inline MaxDims max_dims(int Wa, int Wb, int Wo) {
  MaxDims d;
  d.pp = Wa | 1;
  d.qp = (Wb + 7) | 1;  // at least 7 cells of -inf between two rows of b
  d.q_rows = kMaxRows + Wo - 1;
  d.q_off = (kMmSlack + kMaxRows * d.pp + 2 * (d.pp - Wa) + kMmSlack + 3) & ~3;
  // 8 rows more than staged: the last block of diagonals reaches past Wo
  d.ops_floats = (d.q_off + (d.q_rows + 8) * d.qp + 2 * (d.qp - Wb) + kMmSlack + 3) & ~3;
  // operands | values [64][Wo] and indices [64][Wo]
  const int tile = max(d.ops_floats, 2 * ((kMaxRows * Wo + 3) & ~3));
  d.bytes = sizeof(float) * (size_t)tile;
  return d;
}

__global__ __launch_bounds__(256, 2) void k_band_max_fwd(const BandArgs p, int strips, const MaxDims d,
                                                         long cells_a, long cells_b, int nseg, int Wseg) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int wg = xcd_strip_id();
  const int seg = wg % nseg;  // the segments of a strip run side by side: they share its rows of a
  wg /= nseg;
  const int batch = wg / strips, x0 = (wg - batch * strips) * kMaxRows;
  const int n = p.n, Wa = p.Wa, Wb = p.Wb, Wo = p.Wo, r_lu = p.r_lu;
  const int j_lo = seg * Wseg, Ws = min(Wseg, Wo - j_lo);  // this workgroup's diagonals [j_lo, j_lo + Ws)
  const long bn = (long)batch * n;
  float* PL = smem + kMmSlack;
  float* QL = smem + d.q_off;

  // ---- staging
  const int q0 = x0 - r_lu + j_lo;  // first row of b that the segment's cells meet
  const int qr0 = max(q0, 0), qr1 = min(q0 + d.q_rows, n);
  const int pr1 = min(x0 + kMaxRows, n);
  MmFlat<14, elem_t> sq;
  MmFlat<6, elem_t> sp;
  sq.init(p.b, p.b + cells_b, (bn + qr0) * Wb, (qr1 - qr0) * Wb, Wb, d.qp);
  sq.load(p.b, p.b + cells_b, 0, tid);
  sp.init(p.a, p.a + cells_a, (bn + x0) * Wa, (pr1 - x0) * Wa, Wa, d.pp);
  sp.load(p.a, p.a + cells_a, 0, tid);
  sq.store(QL, 0, tid);
  for (int b = 1; sq.more(b); ++b) {
    sq.load(p.b, p.b + cells_b, b, tid);
    sq.store(QL, b, tid);
  }
  sp.store(PL, 0, tid);
  for (int b = 1; sp.more(b); ++b) {
    sp.load(p.a, p.a + cells_a, b, tid);
    sp.store(PL, b, tid);
  }
  {  // -inf between the rows of b (and before the first): cells that are no k of a cell
    const int gap = d.qp - Wb, first = sq.origin() - (qr0 - q0) * d.qp;
    for (int e = tid; e < (d.q_rows + 1) * gap; e += 256) {
      const int r = e / gap, c = e - r * gap;
      const int at = first + (r - 1) * d.qp + Wb + c;
      if (at >= 0) QL[at] = -INFINITY;
    }
  }
  __syncthreads();
  const int pp = d.pp, qp = d.qp;
  const float* Pt = PL + sp.origin();                        // a[x0 + r][k] = Pt[r * pp + k]
  const float* Qt = QL + sq.origin() - (qr0 - q0) * qp;      // b[q0 + r][k2] = Qt[r * qp + k2]

  // ---- products
  const int x = x0 + lane;
  // every row of the strip is inside the matrix with its whole band, and so is every b row
  const bool interior = x0 >= max(p.a_lu, r_lu) && x0 + kMaxRows - 1 <= n - 1 - max(Wa - 1 - p.a_lu, Wo - 1 - r_lu);
  const float* ap = Pt + lane * pp;
  const int nblocks = (Ws + 7) >> 3;
  float val[5][8];  // blocks wave, wave + 4, ...: at most 5 of them (Ws <= 160)
  int ind[5][8];
#pragma unroll
  for (int s = 0; s < 5; ++s) {
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      val[s][t] = kFloor;
      ind[s][t] = -1;
    }
    const int jb = wave + 4 * s;
    if (jb < nblocks) {
      const int j0 = j_lo + 8 * jb;
      // b[o][k2] of cell t at step k: Qt[(lane + j0 - j_lo + t) * qp + k - j0 - t + Wb - 1]
      const float* bp = Qt + (lane + j0 - j_lo) * qp + (Wb - 1 - j0);
      const int dt = qp - 1;
      auto fold = [&](int t, float av, float bv, int k) __attribute__((always_inline)) {
        const float v = av + bv;
        if (v > val[s][t]) {
          val[s][t] = v;
          ind[s][t] = k;
        }
      };
      if (interior) {
        // all 8 cells walk the union of their k ranges: where a cell has no such k it reads
        // -inf from between the rows
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
            for (int t = 0; t < 8; ++t) fold(t, av[u], bv[u][t], k + u);
        }
        for (; k <= khi; ++k) {
          const float av = ap[k];
#pragma unroll
          for (int t = 0; t < 8; ++t) fold(t, av, bp[t * dt + k], k);
        }
      } else if (x < n) {
        // the reference's k range per cell (k2 in [0, Wb), dense row i + k - lu_a in [0, n))
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          const int j = j0 + t, o = x + j - r_lu;
          if (j < j_lo + Ws && o >= 0 && o < n) {
            const int klo = max(max(0, j - (Wb - 1)), p.a_lu - x), khi = min(min(Wa - 1, j), n - 1 + p.a_lu - x);
            for (int k = klo; k <= khi; ++k) fold(t, ap[k], bp[t * dt + k], k);
          }
        }
      }
    }
  }
  __syncthreads();  // the operands are consumed: their place becomes the result tiles

  float* Sv = smem;
  int* Si = reinterpret_cast<int*>(smem + ((kMaxRows * Ws + 3) & ~3));
#pragma unroll
  for (int s = 0; s < 5; ++s) {
    const int jb = wave + 4 * s;
    if (jb < nblocks) {
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int js = 8 * jb + t, o = x + j_lo + js - r_lu;
        if (js < Ws) {
          const bool inside = x < n && o >= 0 && o < n;  // outside: the reference's zero fill
          Sv[lane * Ws + js] = inside ? val[s][t] : 0.f;
          Si[lane * Ws + js] = inside ? ind[s][t] : 0;
        }
      }
    }
  }
  __syncthreads();

  const int rows = min(kMaxRows, n - x0), cells = rows * Ws;
  elem_t* ob = p.o0 + (bn + x0) * Wo + j_lo;
  int32_t* ib = p.oidx + (bn + x0) * Wo + j_lo;
  typedef int mm_i4 __attribute__((ext_vector_type(4)));
  if (Ws == Wo && (cells & 3) == 0 &&
      ((reinterpret_cast<uintptr_t>(ob) | reinterpret_cast<uintptr_t>(ib)) & 15) == 0) {
    for (int e = 4 * tid; e < cells; e += 1024) {  // the strip's rows are one contiguous run
      st4a(ob + e, *reinterpret_cast<const float4*>(Sv + e));
      *reinterpret_cast<mm_i4*>(ib + e) = *reinterpret_cast<const mm_i4*>(Si + e);
    }
  } else {
    for (int e = tid; e < cells; e += 256) {  // runs of Ws cells, one per row
      const int r = e / Ws, c = e - r * Ws;
      ob[(long)r * Wo + c] = to_elem<elem_t>(Sv[e]);
      ib[(long)r * Wo + c] = Si[e];
    }
  }
}

}  // namespace GENBMM_NS
