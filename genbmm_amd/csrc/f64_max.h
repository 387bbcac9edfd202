// Double-precision max / prod-max products and their arg-max backward (gfx950).
//
// Forward (reference max_cuda_forward_kernel, matmul_cuda_kernel.cu:47-75, and
// prod_max_cuda_forward_kernel, :124-152, instantiated for double by the dispatch at :498-511):
// out[m,n] = max_k a[m,k] (+ or *) b[k,n] with the first k that reaches it - ascending k, strict
// '>', running maximum from -1e9 with index -1.  A workgroup of 256 lanes owns a 64 x 64 tile of
// the result and walks K in slabs of 16 through LDS (a transposed to [k][m], so that both
// operands are read as 16-byte pieces that many lanes share); a lane keeps 4 x 4 running maxima
// in registers, and with each the number of the group of four consecutive k that last raised
// it: per term an add (multiply) and a maximum, per group a compare and a select, instead of a
// compare and three selects per term.  When K is through, every cell forms the four terms of
// its group again, from memory, and keeps the first that equals its maximum - a later group
// only takes over with a strictly larger term, and inside the group the first equal term is
// the one the reference's walk stops at - so value and index are the sequential loop's bit for
// bit.  A NaN term never wins, in the walk (NaN > m is false) as in v_max_f64; k beyond K are
// staged as NaN.  Lanes run along n: the reads of b and the stores of out / idx are contiguous.
//
// Backward (reference :336-456, one thread per gradient cell scanning the whole reduced axis,
// O(M K N)): the scatter of dense_bwd.hip in double precision.  A lane owns a row m of grad_a
// (a column n of grad_b) and kArg64 consecutive k, walks its row in ascending n (its column in
// ascending m) once and adds each term whose index falls into its k to an accumulator in LDS -
// the additions that meet in a cell happen in the reference's order, products are rounded
// before the add, so the sums are bit-identical, in O(M N) work.
#pragma once

#include "common.h"

namespace GENBMM_NS {

typedef double d64x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kD64Tile = 64, kD64Slab = 16, kD64Group = 4, kD64Lda = 66;  // 66: the transposed stores of a half-wave meet no bank twice
constexpr double kD64Floor = -1e9;

template <bool PROD>
__global__ __launch_bounds__(256) void k64_max_fwd(const double* __restrict__ a, const double* __restrict__ b,
                                                  double* __restrict__ out, int32_t* __restrict__ idx, int M,
                                                  int K, int N, int tiles_m, int tiles_n, int vec_o) {
  __shared__ __attribute__((aligned(16))) double As[kD64Slab * kD64Lda];   // [k][m]
  __shared__ __attribute__((aligned(16))) double Bs[kD64Slab * kD64Tile];  // [k][n]
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int per = tiles_m * tiles_n, tile = xcd_renumber(blockIdx.x, gridDim.x);
  const int batch = tile / per, rem = tile - batch * per;
  const int m0 = (rem / tiles_n) * kD64Tile, n0 = (rem % tiles_n) * kD64Tile;
  const double* ab = a + (long)batch * M * K;
  const double* bb = b + (long)batch * K * N;

  // loaders: a - 16 lanes along k, rows ar + 16 i; b - 64 lanes along n, rows bk + 4 i.  Cells
  // beyond M and N belong to results that are not stored; a NaN in a makes a term that never wins.
  const int ak = tid & 15, ar = tid >> 4, bn = tid & 63, bk = tid >> 6;
  double ra[4], rb[4];
  auto gload = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + ar + 16 * i, k = k0 + ak;
      ra[i] = k < K ? (m < M ? ab[(long)m * K + k] : 0.0) : __builtin_nan("");
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + bk + 4 * i, n = n0 + bn;
      rb[i] = (k < K && n < N) ? bb[(long)k * N + n] : 0.0;
    }
  };
  auto sstore = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) As[ak * kD64Lda + ar + 16 * i] = ra[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) Bs[(bk + 4 * i) * kD64Tile + bn] = rb[i];
  };

  double mx[4][4];
  int grp[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      mx[i][j] = kD64Floor;
      grp[i][j] = -1;
    }
  auto term = [](double x, double y) __attribute__((always_inline)) { return PROD ? __dmul_rn(x, y) : __dadd_rn(x, y); };
  // the four steps kk .. kk + 3 of the slab in LDS are group `code`
  auto group = [&](int kk, int code) __attribute__((always_inline)) {
    double av[kD64Group][4], bv[kD64Group][4];
#pragma unroll
    for (int q = 0; q < kD64Group; ++q) {
      const d64x2 a01 = *reinterpret_cast<const d64x2*>(As + (kk + q) * kD64Lda + ty * 4);
      const d64x2 a23 = *reinterpret_cast<const d64x2*>(As + (kk + q) * kD64Lda + ty * 4 + 2);
      const d64x2 b01 = *reinterpret_cast<const d64x2*>(Bs + (kk + q) * kD64Tile + tx * 4);
      const d64x2 b23 = *reinterpret_cast<const d64x2*>(Bs + (kk + q) * kD64Tile + tx * 4 + 2);
      av[q][0] = a01.x, av[q][1] = a01.y, av[q][2] = a23.x, av[q][3] = a23.y;
      bv[q][0] = b01.x, bv[q][1] = b01.y, bv[q][2] = b23.x, bv[q][3] = b23.y;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const double t = __builtin_fmax(__builtin_fmax(term(av[0][i], bv[0][j]), term(av[1][i], bv[1][j])),
                                        __builtin_fmax(term(av[2][i], bv[2][j]), term(av[3][i], bv[3][j])));
        grp[i][j] = t > mx[i][j] ? code : grp[i][j];
        mx[i][j] = __builtin_fmax(mx[i][j], t);
      }
  };
  if (K > 0) gload(0);
  for (int k0 = 0; k0 < K; k0 += kD64Slab) {
    __syncthreads();
    sstore();
    __syncthreads();
    if (k0 + kD64Slab < K) gload(k0 + kD64Slab);
#pragma unroll
    for (int q = 0; q < kD64Slab / kD64Group; ++q) group(q * kD64Group, k0 / kD64Group + q);
  }

  // the first term of the cell's group that equals its maximum: the reference's value and index
  double* ob = out + (long)batch * M * N;
  int32_t* ib = idx + (long)batch * M * N;
  const int n = n0 + tx * 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
    double val[4];
    int ind[4];
    double ta[4][kD64Group], tb[4][kD64Group];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int q = 0; q < kD64Group; ++q) {
        const int k = grp[i][j] * kD64Group + q;
        const bool there = grp[i][j] >= 0 && k < K && n + j < N;
        ta[j][q] = there ? ab[(long)m * K + k] : 0.0;
        tb[j][q] = there ? bb[(long)k * N + n + j] : 0.0;
      }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      val[j] = kD64Floor;
      ind[j] = -1;
#pragma unroll
      for (int q = kD64Group - 1; q >= 0; --q) {  // descending: the lowest k that matches stays
        const int k = grp[i][j] * kD64Group + q;
        const double v = term(ta[j][q], tb[j][q]);
        if (grp[i][j] >= 0 && k < K && v == mx[i][j]) {
          val[j] = v;
          ind[j] = k;
        }
      }
    }
    const long at = (long)m * N + n;
    if (vec_o && n + 3 < N) {
      *reinterpret_cast<d64x2*>(ob + at) = d64x2{val[0], val[1]};
      *reinterpret_cast<d64x2*>(ob + at + 2) = d64x2{val[2], val[3]};
      *reinterpret_cast<i32x4*>(ib + at) = i32x4{ind[0], ind[1], ind[2], ind[3]};
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n + j < N) {
          ob[at + j] = val[j];
          ib[at + j] = ind[j];
        }
    }
  }
}

// ---------------------------------------------------------------- arg-max backward
constexpr int kArg64 = 32;                                    // cells of the reduction axis per lane
constexpr int kArg64Acc = 64 * kArg64 + 64 + 64;              // doubles of LDS: accumulators, row padding, spare cells

// Four ordered additions with one LDS round trip (add4_ordered of common.h in double precision).
__device__ __forceinline__ void add4_ordered(double* __restrict__ accs, const int (&s)[4], const double (&v)[4]) {
  const double r0 = accs[s[0]], r1 = accs[s[1]], r2 = accs[s[2]], r3 = accs[s[3]];
  const double v0 = __dadd_rn(r0, v[0]);
  const double v1 = __dadd_rn(s[1] == s[0] ? v0 : r1, v[1]);
  const double v2 = __dadd_rn(s[2] == s[1] ? v1 : (s[2] == s[0] ? v0 : r2), v[2]);
  const double v3 = __dadd_rn(s[3] == s[2] ? v2 : (s[3] == s[1] ? v1 : (s[3] == s[0] ? v0 : r3)), v[3]);
  accs[s[0]] = v0;
  accs[s[1]] = v1;
  accs[s[2]] = v2;
  accs[s[3]] = v3;
}

// One workgroup of 64 lanes = (64 >> ps) lines x 2^ps parts of kArg64 consecutive k.
// GRAD_A: line = row m, walked along n (stride 1), factor b[k][n], result grad_a[m][k], accumulators
// [line][k] (rows of the result are then contiguous runs).  Otherwise: line = column n, walked along m
// (stride N), factor a[m][k], result grad_b[k][n], accumulators [k][line].
template <bool PROD, bool GRAD_A>
__device__ __forceinline__ void argmax64_block(double* __restrict__ accs, int blk, const double* __restrict__ other,
                                               const int32_t* __restrict__ idx, const double* __restrict__ g,
                                               double* __restrict__ grad, int M, int K, int N, int line_tiles,
                                               int k_chunks, int ps) {
  const int lane = threadIdx.x, parts = 1 << ps, lines = 64 >> ps;
  const int part = lane & (parts - 1), line = lane >> ps;
  const int spare = 64 * kArg64 + 64 + lane;
  const int kc_id = blk % k_chunks, lt = blk / k_chunks;
  const int batch = lt / line_tiles;
  const int l0 = (lt - batch * line_tiles) * lines, l = l0 + line;
  const int kw = parts * kArg64;                       // k covered by the workgroup
  const int w0 = kc_id * kw, c0 = w0 + part * kArg64;  // first k of the workgroup / of this lane
  const int kc = min(kArg64, K - c0);                  // <= 0: the part lies beyond K
  const int L = GRAD_A ? M : N, W = GRAD_A ? N : M;    // lines of the gradient / cells walked per line
  const bool live = l < L;
  const int ll = live ? l : 0;
  const long first = GRAD_A ? ((long)batch * M + ll) * N : (long)batch * M * N + ll, step = GRAD_A ? 1 : N;
  const int32_t* iw = idx + first;
  const double* gw = g + first;
  const double* ob = PROD ? (GRAD_A ? other + (long)batch * K * N : other + (long)batch * M * K) : nullptr;
  const int base = GRAD_A ? line * (kw + 1) + part * kArg64 : (part * kArg64) * lines + line;
  const int pitch = GRAD_A ? 1 : lines;
  for (int kk = 0; kk < kArg64; ++kk) accs[base + kk * pitch] = 0.0;
  accs[spare] = 0.0;
  auto slot = [&](int ki) __attribute__((always_inline)) {
    const int k = ki - c0;
    return (k >= 0 && k < kc) ? base + k * pitch : spare;
  };
  // the term of cell w: g, times the other operand at the cell's index for the product semiring
  // (read only when the index falls into this lane's k)
  auto term = [&](int w, int ki, double gv) __attribute__((always_inline)) {
    const int k = ki - c0;
    if (PROD && k >= 0 && k < kc) return __dmul_rn(GRAD_A ? ob[(long)ki * N + w] : ob[(long)w * K + ki], gv);
    return gv;
  };
  if (live) {
    int w = 0;
    for (; w + 8 <= W; w += 8) {
      int iv[8];
      double gv[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        iv[q] = iw[(long)(w + q) * step];
        gv[q] = gw[(long)(w + q) * step];
      }
#pragma unroll
      for (int q = 0; q < 8; ++q) gv[q] = term(w + q, iv[q], gv[q]);
#pragma unroll
      for (int q = 0; q < 8; q += 4) {
        const int sl[4] = {slot(iv[q]), slot(iv[q + 1]), slot(iv[q + 2]), slot(iv[q + 3])};
        const double tv[4] = {gv[q], gv[q + 1], gv[q + 2], gv[q + 3]};
        add4_ordered(accs, sl, tv);
      }
    }
    for (; w < W; ++w) {
      const int ki = iw[(long)w * step], s = slot(ki);
      accs[s] = __dadd_rn(accs[s], term(w, ki, gw[(long)w * step]));
    }
  }
  __syncthreads();
  const int nl = min(lines, L - l0), kn = min(kw, K - w0);
  if (GRAD_A) {
    for (int r = 0; r < nl; ++r) {
      double* dst = grad + ((long)batch * M + l0 + r) * K + w0;
      for (int kk = lane; kk < kn; kk += 64) dst[kk] = accs[r * (kw + 1) + kk];
    }
  } else {
    const int lc = lane & (lines - 1), lk = lane / lines;
    if (lc < nl)
      for (int kk = lk; kk < kn; kk += parts) grad[((long)batch * K + w0 + kk) * N + l0 + lc] = accs[kk * lines + lc];
  }
}

// Both gradients in one launch, batch item by batch item (ta workgroups of grad_a, then tb of
// grad_b; XCD-aware numbering): both read the item's idx and g.
template <bool PROD>
__global__ __launch_bounds__(64) void k64_argmax_bwd_both(const double* __restrict__ amat, const double* __restrict__ bmat,
                                                         const int32_t* __restrict__ idx, const double* __restrict__ g,
                                                         double* __restrict__ grad_a, double* __restrict__ grad_b, int M,
                                                         int K, int N, int row_tiles, int kc_a, int ps_a, int col_tiles,
                                                         int kc_b, int ps_b) {
  __shared__ double accs[kArg64Acc];
  const int ta = row_tiles * kc_a, tb = col_tiles * kc_b;
  const int v = xcd_renumber(blockIdx.x, gridDim.x);
  const int item = v / (ta + tb), r = v - item * (ta + tb);
  if (r < ta)
    argmax64_block<PROD, true>(accs, item * ta + r, bmat, idx, g, grad_a, M, K, N, row_tiles, kc_a, ps_a);
  else
    argmax64_block<PROD, false>(accs, item * tb + r - ta, amat, idx, g, grad_b, M, K, N, col_tiles, kc_b, ps_b);
}

}  // namespace GENBMM_NS
