// Strip kernels for the banded (+,*) and log products: the operands of a strip
// of 64 matrix columns are staged through LDS, so every band element is read
// from memory once per strip (plus the halo of the sliding operand) and every
// load and store is a run along the band axis.
//
// Walking the diagonals.  With k2 = k - j + (Wb - 1) independent of i,
//   forward   out[i,j]  = sum_k  a[i,k]       * b[i+j-lu_o, k-j+Wb-1]
//   grad_a    ga[i,k]   = sum_j  g'[i,j]      * b[i+j-lu_o, k-j+Wb-1]
//   grad_b    gb[o,k2]  = sum_j  g'[o-j+lu_o,j] * a[o-j+lu_o, k2+j-(Wb-1)]
// a lane owns one row (i, resp. o) and a block of 8 adjacent outputs along the
// band axis (j, k, k2); one step of the sum reads one value of the lane's own
// row and 8 values of the other operand, which sit on an anti-diagonal of its
// LDS tile: row + 1, column - 1 per output.  Row strides are odd, so the 64
// lanes of a wave (64 consecutive rows) hit 64 different banks at every step.
// The other operand's rows carry 7 cells of padding on both sides holding the
// semiring zero, and matrix-edge cells are zeroed while staging, so the inner
// loop has no predicates.  The band axis of the sum/outputs is cut into chunks
// of 32 (8 per wave); the sliding operand's 64 + 31 rows are re-staged per chunk.
//
// Log semiring: factored like the dense logbmm.  alpha[i] = max_k a[i,k],
// beta[o] = max_k2 b[o,k2] (over the cells inside the matrix) are taken by the
// wave that stages the row, the tiles hold exp(a - alpha), exp(b - beta) and
// the sum is a multiply-add; out = log S + alpha + beta.  The backward stages
// H = g * exp(alpha + beta - out) in place of g.  A cell whose S falls below
// 2^-40 (forward) or whose alpha + beta - out exceeds 40 ln 2 (backward) is
// recomputed - the cell, resp. the gradient rows it feeds - by the per-cell
// routine from global memory.
#pragma once

#include "banded_cells.h"

namespace GENBMM_NS {

constexpr int kBT = 64;              // rows per strip = lanes of a wave
constexpr int kBJ = 32;              // band-axis chunk: 4 waves x 8
constexpr int kBR = kBT + kBJ - 1;   // rows of the sliding operand per chunk
constexpr int kBP = 7;               // padding cells on both sides of its rows
constexpr int kBC = kBJ + 1;         // row stride of the output staging tile
constexpr float kBandGuardBits = 40.f;

struct StripDims {
  int ld_own;    // row stride of the lane's own operand tile
  int ld_sl;     // row stride of the sliding operand tile (padded)
  size_t bytes;  // dynamic LDS
};

inline int odd(int x) { return x | 1; }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Staging of `ROWS` rows of a band operand (width W, lu given) starting at
// matrix column row0 into tile[r * ld + pad + k]; columns [0, pad) and
// [pad + W, ld) and every cell outside the matrix get the semiring zero.  LOG:
// the tile gets exp(x - rowmax) and shift[r] the row maximum (over cells inside
// the matrix).  One wave per row (rows wave, wave+4, ...), lanes along the band
// axis, NQ = ceil(ld / 64) cells per lane.  load() only issues the global
// loads into registers, store() consumes them - a whole chunk is in flight while
// the previous one is being multiplied.
constexpr int kSemMul = 0, kSemLog = 1, kSemMax = 2;  // what a staged tile is used for
constexpr int kSemLogPrep = 3;  // log product on operands prepared by k_band_prep (forward kernel only)

template <int SEM, int NQ, int ROWS>
struct RowStage {
  static constexpr bool LOG = SEM == kSemLog;
  static constexpr int U = (ROWS + 3) / 4;
  float v[U][NQ];

  // E: float (a workspace) or the element type of the caller's tensors (widened here)
  template <class E>
  __device__ __forceinline__ void load(const E* __restrict__ src, int W, int lu, int n, int row0,
                                       int ld, int pad, int wave, int lane) {
    const float fill = SEM == kSemMul ? 0.f : -INFINITY;
    // Strips away from the matrix edges (all but a few per batch item): every staged
    // row exists and every band cell of it lies inside the matrix, so the only
    // predicate left is the lane's own column - one masked region per q instead of
    // five comparisons per element.
    const bool interior = row0 - lu >= 0 && row0 + ROWS + W - 2 - lu <= n - 1;  // uniform
    if (interior) {
      const E* base = src + (long)(row0 + wave) * W - pad + lane;
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const int col = lane + 64 * q, k = col - pad;
        const bool kin = col < ld && k >= 0 && k < W;
#pragma unroll
        for (int u = 0; u < U; ++u) v[u][q] = fill;
        if (kin) {
#pragma unroll
          for (int u = 0; u < U; ++u)
            if (4 * u + 3 < ROWS || wave + 4 * u < ROWS) v[u][q] = base[(long)(4 * u) * W + 64 * q];
        }
      }
      return;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = wave + 4 * u, c = row0 + r;  // c: matrix column = row of the band tensor
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const int col = lane + 64 * q, k = col - pad;
        const int prow = c + k - lu;  // dense row of this cell
        const bool ok = r < ROWS && col < ld && c >= 0 && c < n && k >= 0 && k < W && prow >= 0 && prow < n;
        v[u][q] = ok ? src[(long)c * W + k] : fill;
      }
    }
  }

  __device__ __forceinline__ void store(float* __restrict__ tile, int ld, float* __restrict__ shift,
                                        int wave, int lane) const {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = wave + 4 * u;
      if (r < ROWS) {
        float m = 0.f;
        if (LOG) {
          m = v[u][0];
#pragma unroll
          for (int q = 1; q < NQ; ++q) m = fmaxf(m, v[u][q]);
          m = wave_max(m);
          if (lane == 0) shift[r] = m;
          if (m == -INFINITY) m = 0.f;  // row without a cell inside the matrix: all zeros
        }
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          const int col = lane + 64 * q;
          if (tile && col < ld) tile[r * ld + col] = LOG ? fast_exp2((v[u][q] - m) * kLog2e) : v[u][q];
        }
      }
    }
  }
};

// ------------------------------------------------------------ prepared operands
// Four lanes per band row: shift = maximum over the cells inside the matrix (-inf if
// there is none), e = exp(x - shift), 0 for cells outside.  With these the log
// product is a (+,x) product of e's plus an epilogue, and no kernel downstream
// takes an exponential per staged element again.
// Both operands in one launch.  A workgroup takes R consecutive band rows of one operand -
// one contiguous block of memory, moved 16 bytes per lane in both directions - and turns them
// in LDS (row stride ld, odd) so that 256 / R lanes share a row.
struct PrepSide {
  const elem_t* x;
  float* e;
  float* shift;
  int W, lu, ld;
};
constexpr int kPrepRows = 64;  // measured against 128 and 256: the row pass is the slow part, and
                               // it is faster with four lanes to a row

template <int R>
__device__ __forceinline__ void band_prep_block(const PrepSide& q, float* __restrict__ tile, int n, long rows,
                                                long row0, int vec) {
  constexpr int PARTS = 256 / R;
  const int tid = threadIdx.x, W = q.W, ld = q.ld;
  const int nr = (int)min((long)R, rows - row0);
  const int cells = nr * W;
  const elem_t* xb = q.x + row0 * W;
  float* eb = q.e + row0 * W;
  constexpr int U = 8;
  // Index arithmetic is what this kernel would otherwise spend its time on: the LDS offset of a
  // lane's 16-byte piece advances by a fixed step with one carry, and each of its four cells
  // adds the row gap if it lies past the row end - no division, no branch.
  const int quads = (vec && W >= 4) ? cells >> 2 : 0;  // W >= 4: a piece straddles at most one row end
  const int dr = 1024 / W, dk = 1024 - dr * W;        // 256 lanes x 4 cells between a lane's pieces
  const int gap = ld - W, step = dr * ld + dk;
  const int r_first = (4 * tid) / W, k_first = 4 * tid - r_first * W;
  {
    int k = k_first, base = r_first * ld + k_first;  // base: LDS offset of the piece's first cell
    for (int i0 = tid; i0 < quads; i0 += 256 * U) {
      float4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (i0 + 256 * u < quads) v[u] = ld4a(xb + 4 * (i0 + 256 * u));
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (i0 + 256 * u < quads) {
          tile[base] = v[u].x;
          tile[base + 1 + (k + 1 >= W ? gap : 0)] = v[u].y;
          tile[base + 2 + (k + 2 >= W ? gap : 0)] = v[u].z;
          tile[base + 3 + (k + 3 >= W ? gap : 0)] = v[u].w;
        }
        k += dk;
        base += step;
        if (k >= W) {
          k -= W;
          base += gap;
        }
      }
    }
    for (int i = 4 * quads + tid; i < cells; i += 256) tile[(i / W) * ld + i % W] = xb[i];
  }
  __syncthreads();
  {
    const int r = tid / PARTS, part = tid % PARTS;
    const int per = (W + PARTS - 1) / PARTS, k0 = part * per, k1 = min(W, k0 + per);
    const bool live = r < nr;
    const int c = live ? (int)((unsigned)((row0 + r) % n)) : 0;
    // cells of this lane's share that lie inside the matrix: k in [lo, hi)
    const int lo = max(k0, max(0, q.lu - c)), hi = live ? min(k1, min(W - 1, n - 1 + q.lu - c) + 1) : lo;
    float* tr = tile + r * ld;
    float m = -INFINITY;
    // every lane walks its whole share (a uniform trip count); cells outside take no part
#pragma unroll 4
    for (int k = k0; k < k0 + per; ++k) {
      const bool in = k >= lo && k < hi;
      const float x = tr[in ? k : 0];
      m = in ? fmaxf(m, x) : m;
    }
#pragma unroll
    for (int o = 1; o < PARTS; o <<= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    if (live && part == 0) q.shift[row0 + r] = m;
    const float sh = m == -INFINITY ? 0.f : m;
#pragma unroll 4
    for (int k = k0; k < k0 + per; ++k) {
      const bool in = k >= lo && k < hi;
      const float e = fast_exp2((tr[in ? k : 0] - sh) * kLog2e);
      if (live && k < k1) tr[k] = in ? e : 0.f;
    }
  }
  __syncthreads();
  {
    int k = k_first, base = r_first * ld + k_first;
    for (int i = tid; i < quads; i += 256) {
      const float4 w = make_float4(tile[base], tile[base + 1 + (k + 1 >= W ? gap : 0)],
                                   tile[base + 2 + (k + 2 >= W ? gap : 0)], tile[base + 3 + (k + 3 >= W ? gap : 0)]);
      *reinterpret_cast<float4*>(eb + 4 * i) = w;
      k += dk;
      base += step;
      if (k >= W) {
        k -= W;
        base += gap;
      }
    }
    for (int i = 4 * quads + tid; i < cells; i += 256) eb[i] = tile[(i / W) * ld + i % W];
  }
}

// Workgroups [0, blocks_a) take the first operand, the rest the second.
__global__ __launch_bounds__(256) void k_band_prep(const PrepSide pa, const PrepSide pb, int n, long rows,
                                                   int blocks_a, int vec) {
  extern __shared__ __attribute__((aligned(16))) float tile[];
  const bool first = (int)blockIdx.x < blocks_a;
  const long row0 = (long)(first ? blockIdx.x : blockIdx.x - blocks_a) * kPrepRows;
  band_prep_block<kPrepRows>(first ? pa : pb, tile, n, rows, row0, vec);
}

// ------------------------------------------------------------------ forward
// Workgroup ids are dealt round-robin to the 8 XCDs (one L2 each): renumber so
// that an XCD works on consecutive strips, whose halos overlap.
__device__ __forceinline__ int xcd_strip_id() { return xcd_renumber(blockIdx.x, gridDim.x); }

// The exact recompute of one cell, kept out of line: it is rare, and inlined it costs
// the strip kernels registers they do not have.
__device__ __forceinline__ float band_fwd_cell_log_exact(const BandArgs& p, long bi, int i, int j) {
  band_fwd_cell<GENBMM_BAND_LOG>(p, bi, i, j);
  return p.o0[bi * p.Wo + j];
}
// Out of line for the wide-band variants of the strip kernels, which have no registers to
// spare for it (the narrow ones take it inline: a call costs every lane a stack frame).
__device__ __attribute__((noinline)) float band_fwd_cell_log_exact_call(const BandArgs& p, long bi, int i, int j) {
  return band_fwd_cell_log_exact(p, bi, i, j);
}

template <int SEM, int NQ>
__global__ __launch_bounds__(256, (SEM == kSemMul || SEM == kSemLogPrep) ? 3 : 2) void k_band_fwd_strip(const BandArgs p, int strips,
                                                                          int ld_own, int ld_sl) {
  constexpr bool LOG = SEM == kSemLog, MAXP = SEM == kSemMax, PREP = SEM == kSemLogPrep;
  constexpr int SS = PREP ? kSemMul : SEM;  // how the tiles are staged
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float* As = smem;                 // [64][ld_own]
  float* Bs = As + kBT * ld_own;    // [95][ld_sl]; reused as the [64][33] output staging tile
  float* al = Bs + kBR * ld_sl;     // [64]
  float* be = al + kBT;             // [95]
  float* Cs = Bs;
  int* Is = reinterpret_cast<int*>(Bs + kBT * kBC);  // max product: the argmax tile behind it
  float* Rt = Bs + kBT * kBC;                        // prepared log product: the 1/S tile
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wg = xcd_strip_id();
  const int batch = wg / strips, i0 = (wg - batch * strips) * kBT;
  const int n = p.n, Wa = p.Wa, Wb = p.Wb, Wo = p.Wo;
  // the prepared product reads the workspace's factors (float), the others the caller's tensors
  auto ab = [&] {
    if constexpr (PREP) return static_cast<const float*>(p.ws_ea) + (long)batch * n * Wa;
    else return p.a + (long)batch * n * Wa;
  }();
  auto bb = [&] {
    if constexpr (PREP) return static_cast<const float*>(p.ws_eb) + (long)batch * n * Wb;
    else return p.b + (long)batch * n * Wb;
  }();
  elem_t* ob = p.o0 + (long)batch * n * Wo;
  int32_t* ib = MAXP ? p.oidx + (long)batch * n * Wo : nullptr;
  float* rb = PREP ? p.ws_r + (long)batch * n * Wo : nullptr;
  const long bn = (long)batch * n;
  const float thr = fast_exp2(-kBandGuardBits);

  {
    RowStage<SS, NQ, kBT> sa;
    sa.load(ab, Wa, p.a_lu, n, i0, ld_own, 0, wave, lane);
    sa.store(As, ld_own, al, wave, lane);
  }
  float* bw = be + kBR;  // prepared log product: beta[i0 - lu_out + t], t < 64 + Wo (+ chunk round-up)
  if (PREP) {
    if (tid < kBT) al[tid] = i0 + tid < n ? p.ws_al[bn + i0 + tid] : 0.f;
    for (int t = tid; t < kBT + Wo + kBJ; t += 256) {
      const int o = i0 - p.r_lu + t;
      bw[t] = (o >= 0 && o < n) ? p.ws_be[bn + o] : 0.f;
    }
  }
  RowStage<SS, NQ, kBR> sb;
  sb.load(bb, Wb, p.b_lu, n, i0 - p.r_lu, ld_sl, kBP, wave, lane);

  for (int jc = 0; jc < Wo; jc += kBJ) {
    __syncthreads();  // the previous chunk's output tile has been written out
    sb.store(Bs, ld_sl, be, wave, lane);
    __syncthreads();
    if (jc + kBJ < Wo) sb.load(bb, Wb, p.b_lu, n, i0 + jc + kBJ - p.r_lu, ld_sl, kBP, wave, lane);

    const int j0 = jc + 8 * wave;
    // acc: the sum; max product: the running maximum (strictly above the reference's
    // -1e9 floor to count) and its k, lowest k on ties since k ascends
    float acc[8];
    int ind[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      acc[t] = MAXP ? kFloor : 0.f;
      ind[t] = -1;
    }
    auto fold = [&](int t, float av, float bv, int k) __attribute__((always_inline)) {
      if (MAXP) {
        const float v = av + bv;
        if (v > acc[t]) {
          acc[t] = v;
          ind[t] = k;
        }
      } else {
        acc[t] = __builtin_fmaf(av, bv, acc[t]);
      }
    };
    if (j0 < Wo) {
      const int klo = max(0, j0 - (Wb - 1)), khi = min(Wa - 1, j0 + 7);
      const float* ap = As + lane * ld_own;
      // element (t, k): Bs[(lane + 8*wave + t)][k - j0 - t + Wb - 1 + pad]
      const float* bp = Bs + (lane + 8 * wave) * ld_sl + (Wb - 1 + kBP - j0);
      const int dt = ld_sl - 1;
      int k = klo;
      for (; k + 3 <= khi; k += 4) {
        float av[4], bv[4][8];
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          av[x] = ap[k + x];
#pragma unroll
          for (int t = 0; t < 8; ++t) bv[x][t] = bp[t * dt + k + x];
        }
#pragma unroll
        for (int x = 0; x < 4; ++x)
#pragma unroll
          for (int t = 0; t < 8; ++t) fold(t, av[x], bv[x][t], k + x);
      }
      for (; k <= khi; ++k) {
        const float av = ap[k];
#pragma unroll
        for (int t = 0; t < 8; ++t) fold(t, av, bp[t * dt + k], k);
      }
    }
    float sh[8];
    if (LOG) {
#pragma unroll
      for (int t = 0; t < 8; ++t) sh[t] = al[lane] + be[min(lane + 8 * wave + t, kBR - 1)];
    }
    if (PREP) {  // alpha[i] + beta[o], o = i + j - lu_out, staged once per strip
#pragma unroll
      for (int t = 0; t < 8; ++t) sh[t] = al[lane] + bw[lane + j0 + t];
    }
    __syncthreads();  // every wave is done with Bs: it becomes the output tile
    const int i = i0 + lane;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      float v = acc[t];
      if (LOG || PREP) {
        const int j = j0 + t, o = i + j - p.r_lu;
        float rv = 0.f;
        if (i < n && j < Wo && o >= 0 && o < n) {
          if ((v >= thr) && (v < INFINITY) && (sh[t] >= kFloor) && (sh[t] < INFINITY)) {
            rv = __builtin_amdgcn_rcpf(v);
            v = __builtin_fmaf(fast_log2(v), kLn2, sh[t]);
          } else {  // factoring not exact for this cell: recompute it from memory
            v = NQ == 1 ? band_fwd_cell_log_exact(p, bn + i, i, j) : band_fwd_cell_log_exact_call(p, bn + i, i, j);
            rv = -1.f;  // tells the backward that 1/S is not usable here
          }
        } else {
          v = 0.f;  // outside the matrix: the reference's zero fill
        }
        if (PREP) Rt[lane * kBC + 8 * wave + t] = rv;
      }
      if (MAXP) {
        const int o = i + j0 + t - p.r_lu;
        const bool inside = o >= 0 && o < n;
        if (!inside) v = 0.f;  // outside the matrix: the reference's zero fill (index 0 too)
        Is[lane * kBC + 8 * wave + t] = inside ? ind[t] : 0;
      }
      Cs[lane * kBC + 8 * wave + t] = v;
    }
    __syncthreads();
    // rows of 32 consecutive outputs
    for (int e = tid; e < kBT * kBJ; e += 256) {
      const int r = e >> 5, c = e & 31;
      if (i0 + r < n && jc + c < Wo) {
        ob[(long)(i0 + r) * Wo + jc + c] = to_elem<elem_t>(Cs[r * kBC + c]);
        if (MAXP) ib[(long)(i0 + r) * Wo + jc + c] = Is[r * kBC + c];
        if (PREP) rb[(long)(i0 + r) * Wo + jc + c] = Rt[r * kBC + c];
      }
    }
  }
}

// ----------------------------------------------------------------- backward
// Shared by both gradients: the lane owns row x of the OUTPUT operand (a for
// grad_a, b for grad_b) and up to kMaxKB blocks of 8 cells along its band axis;
// per chunk of 32 result diagonals j it multiplies one value of g' (g, or
// H = g*exp(alpha+beta-out) in the log semiring) with 8 values of the other
// operand on an anti-diagonal of its tile.
//   grad_a: g'[x][j]            * b'[x + j - lu_o][kk - j + Wb - 1]
//   grad_b: g'[x - j + lu_o][j] * a'[x - j + lu_o][kk + j - (Wb - 1)]
// The g' tile of one chunk of 32 diagonals: rows x of g (grad_a, 64 rows) or rows
// x - j + lu_o (grad_b, 95 rows).  load() issues all global reads of g (and out)
// of the tile, store() turns them into g' = g (or H = g * exp(alpha + beta - out))
// in LDS.  A cell
// counts if it lies inside the matrix and, for grad_b, if its b row is in the strip.
template <bool LOG, bool GRAD_A, bool PREP = false>
struct GStage {
  static constexpr int ROWS = GRAD_A ? kBT : kBR;
  static constexpr int PER = (ROWS * kBJ + 255) / 256;
  float gv[PER], ov[PER];
  unsigned used;

  // [U0, U1): the pieces handled by this call (all of them, or a few at a time where
  // registers are short)
  template <int U0 = 0, int U1 = PER, class G, class O>
  __device__ __forceinline__ void load(const G* __restrict__ gb, const O* __restrict__ ob,
                                       int x0, int yb, int jc, int n, int Wo, int r_lu, int tid) {
    if (U0 == 0) used = 0;
#pragma unroll
    for (int u = U0; u < (U1 < PER ? U1 : PER); ++u) {
      const int e = tid + 256 * u, r = e >> 5, c = e & 31, j = jc + c;
      const int i = GRAD_A ? x0 + r : yb + r;  // row of g / out (a's row index)
      const int o = i + j - r_lu;              // b's row index of this cell
      const bool inside = r < ROWS && i >= 0 && i < n && j < Wo && o >= 0 && o < n;
      const bool use = inside && (GRAD_A || (o >= x0 && o < x0 + kBT));
      gv[u] = use ? gb[(long)i * Wo + j] : 0.f;
      ov[u] = (LOG && use) ? ob[(long)i * Wo + j] : 0.f;
      used |= (use ? 1u : 0u) << u;
    }
  }

  template <int U0 = 0, int U1 = PER>
  __device__ __forceinline__ void store(float* __restrict__ gt, const float* __restrict__ sh_own,
                                        const float* __restrict__ sh_sl, int* __restrict__ badrow,
                                        int x0, int yb, int jc, int r_lu, float lim, int tid) const {
#pragma unroll
    for (int u = U0; u < (U1 < PER ? U1 : PER); ++u) {
      const int e = tid + 256 * u, r = e >> 5, c = e & 31;
      if (r >= ROWS) continue;
      float v = gv[u];
      if (PREP && v != v) {  // H is NaN: the cell's 1/S is not usable (or g is NaN), the row is redone
        const int o = (GRAD_A ? x0 + r : yb + r) + jc + c - r_lu;
        badrow[GRAD_A ? r : o - x0] = 1;
        v = 0.f;
      }
      if (LOG && ((used >> u) & 1u)) {
        const int o = (GRAD_A ? x0 + r : yb + r) + jc + c - r_lu;
        // alpha[i] + beta[o] - out[i,j]
        const float sa = GRAD_A ? sh_own[r] : sh_sl[r];
        const float sb = GRAD_A ? sh_sl[r + c] : sh_own[o - x0];
        const float ex = sa + sb - ov[u];
        if (!(ex <= lim)) badrow[GRAD_A ? r : o - x0] = 1;  // factoring not exact: row redone
        v *= fast_exp2(ex * kLog2e);
      }
      gt[r * kBC + c] = v;
    }
  }
};

constexpr int kMaxKB = 3;  // band-axis blocks of 8 per wave: widths up to 96

// H = g * R for the prepared log backward, once for both gradients; R < 0 marks a
// cell that the forward computed exactly (its 1/S is not usable): NaN there, which
// the gradient kernels turn into "redo this row exactly".
__global__ __launch_bounds__(256) void k_band_h(const elem_t* __restrict__ g,
                                               const float* __restrict__ r,
                                               float* __restrict__ h, long cells) {
  const long stride = (long)gridDim.x * 1024;
  for (long e = (long)blockIdx.x * 1024 + threadIdx.x; e < cells; e += stride) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const long i = e + 256 * u;
      if (i < cells) {
        const float rv = r[i];
        h[i] = rv < 0.f ? __builtin_nanf("") : (float)g[i] * rv;
      }
    }
  }
}

// PREP (with LOG = false): the log product on the forward's workspace - operands
// EA / EB staged like a (+,x) product, g' = H = g * R from k_band_h, result times
// the own operand's EA / EB; rows fed by a cell whose H is NaN are recomputed exactly.
template <bool LOG, bool GRAD_A, int NQ, bool PREP = false>
__global__ __launch_bounds__(256, 3) void k_band_bwd_strip(const BandArgs p, int strips, int ld_own,
                                                           int ld_sl, int sl_floats) {
  static_assert(!(LOG && PREP), "");
  extern __shared__ __attribute__((aligned(16))) float smem[];
  // sl : 95 rows of the other operand, padded (LOG: exp(y - shift)); reused as the
  //      [64][ld_own] result tile at the end
  // gt : g' tile; grad_a [64][33] (row x), grad_b [95][33] (row x - j + lu_o)
  // The output operand itself is only needed for its row maxima (LOG) and, in the
  // epilogue, as the factor exp(x - shift), which is taken while the rows are
  // written out.
  float* sl = smem;
  float* gt = sl + sl_floats;      // sl_floats = max(95 * ld_sl, 64 * ld_own)
  float* sh_own = gt + kBR * kBC;  // [64] shift of the lane's own row
  float* sh_sl = sh_own + kBT;     // [95] shifts of the staged other-operand rows
  int* badrow = reinterpret_cast<int*>(sh_sl + kBR);  // [64]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wg = xcd_strip_id();
  const int batch = wg / strips, x0 = (wg - batch * strips) * kBT;
  const int n = p.n, Wa = p.Wa, Wb = p.Wb, Wo = p.Wo;
  const long bn = (long)batch * n;
  // the prepared product reads the workspace (float), the others the caller's tensors
  auto ab = [&] {
    if constexpr (PREP) return static_cast<const float*>(p.ws_ea) + bn * Wa;
    else return p.a + bn * Wa;
  }();
  auto bb = [&] {
    if constexpr (PREP) return static_cast<const float*>(p.ws_eb) + bn * Wb;
    else return p.b + bn * Wb;
  }();
  auto gb = [&] {  // PREP: H = g / S, staged once for both gradients
    if constexpr (PREP) return static_cast<const float*>(p.ws_h) + bn * Wo;
    else return p.g + bn * Wo;
  }();
  const elem_t* ob = LOG ? p.out + bn * Wo : nullptr;
  // output operand / other operand
  auto xo = GRAD_A ? ab : bb;
  auto yo = GRAD_A ? bb : ab;
  const int Wx = GRAD_A ? Wa : Wb, Wy = GRAD_A ? Wb : Wa;
  const int lux = GRAD_A ? p.a_lu : p.b_lu, luy = GRAD_A ? p.b_lu : p.a_lu;
  elem_t* gradb = (GRAD_A ? p.o0 : p.o1) + bn * Wx;
  const float lim = kBandGuardBits * kLn2 + 1e-3f;

  if (tid < kBT) badrow[tid] = 0;
  if (LOG) {
    RowStage<kSemLog, NQ, kBT> so;
    so.load(xo, Wx, lux, n, x0, ld_own, 0, wave, lane);
    so.store(nullptr, ld_own, sh_own, wave, lane);  // row maxima only
  }
  float acc[kMaxKB][8];
#pragma unroll
  for (int q = 0; q < kMaxKB; ++q)
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[q][t] = 0.f;

  // first row of the other operand needed by chunk jc
  auto row0_of = [&](int jc) { return GRAD_A ? x0 + jc - p.r_lu : x0 - jc - (kBJ - 1) + p.r_lu; };
  RowStage<LOG ? kSemLog : kSemMul, NQ, kBR> ss;
  ss.load(yo, Wy, luy, n, row0_of(0), ld_sl, kBP, wave, lane);

  for (int jc = 0; jc < Wo; jc += kBJ) {
    const int yb = row0_of(jc);
    __syncthreads();  // previous chunk fully consumed
    ss.store(sl, ld_sl, sh_sl, wave, lane);
    __syncthreads();  // sh_sl visible
    if (jc + kBJ < Wo) ss.load(yo, Wy, luy, n, row0_of(jc + kBJ), ld_sl, kBP, wave, lane);
    // ---- g' tile.  (Starting these reads one chunk ahead, like the operand rows,
    // measured slower: the extra live registers cost more than the latency.)
    // The log kernels are short of registers: they go element by element.
    if (LOG) {
      for (int e = tid; e < GStage<LOG, GRAD_A>::ROWS * kBJ; e += 256) {
        const int r = e >> 5, c = e & 31, j = jc + c;
        const int i = GRAD_A ? x0 + r : yb + r;
        const int o = i + j - p.r_lu;
        const bool inside = i >= 0 && i < n && j < Wo && o >= 0 && o < n;
        float v = 0.f;
        if (inside && (GRAD_A || (o >= x0 && o < x0 + kBT))) {
          const float sa = GRAD_A ? sh_own[r] : sh_sl[r];
          const float sb = GRAD_A ? sh_sl[r + c] : sh_own[o - x0];
          const float ex = sa + sb - (float)ob[(long)i * Wo + j];  // alpha[i] + beta[o] - out[i,j]
          if (!(ex <= lim)) badrow[GRAD_A ? r : o - x0] = 1;  // factoring not exact: row redone
          v = (float)gb[(long)i * Wo + j] * fast_exp2(ex * kLog2e);
        }
        gt[r * kBC + c] = v;
      }
    } else {
      GStage<LOG, GRAD_A, PREP> gs;
      gs.load(gb, ob, x0, yb, jc, n, Wo, p.r_lu, tid);
      gs.store(gt, sh_own, sh_sl, badrow, x0, yb, jc, p.r_lu, lim, tid);
    }
    __syncthreads();
    // ---- multiply
#pragma unroll
    for (int q = 0; q < kMaxKB; ++q) {
      const int k0 = 8 * (wave + 4 * q);  // first band cell of this block
      if (k0 >= Wx) break;
      // j range (within the chunk) that can meet cells k0 .. k0+7
      int jlo, jhi;
      if (GRAD_A) {  // k2 = k - j + Wb - 1 in [0, Wb)
        jlo = max(jc, k0);
        jhi = min(min(jc + kBJ - 1, Wo - 1), k0 + 7 + Wb - 1);
      } else {       // k = k2 + j - (Wb - 1) in [0, Wa)
        jlo = max(jc, Wb - 1 - k0 - 7);
        jhi = min(min(jc + kBJ - 1, Wo - 1), Wb - 1 - k0 + Wa - 1);
      }
      const float* gp;
      const float* yp;
      int gstep, ystep;
      if (GRAD_A) {
        // g'[lane][jj], b'[lane + jj][k0 + t - (jc + jj) + Wb - 1 + pad]
        gp = gt + lane * kBC;
        gstep = 1;
        yp = sl + lane * ld_sl + (k0 - jc + Wb - 1 + kBP);
        ystep = ld_sl - 1;
      } else {
        // row r = lane - jj + 31: g'[r][jj], a'[r][k0 + t + (jc + jj) - (Wb - 1) + pad]
        gp = gt + (lane + kBJ - 1) * kBC;
        gstep = 1 - kBC;
        yp = sl + (lane + kBJ - 1) * ld_sl + (k0 + jc - (Wb - 1) + kBP);
        ystep = 1 - ld_sl;
      }
      for (int j = jlo; j <= jhi; ++j) {
        const int jj = j - jc;
        const float gv = gp[jj * gstep];
        const float* yr = yp + jj * ystep;
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[q][t] = __builtin_fmaf(gv, yr[t], acc[q][t]);
      }
    }
  }

  // ---- epilogue: grad = (LOG ? exp(x - shift) : PREP ? EX : 1) * acc, staged for row-wise
  // stores.  The own operand's rows are requested before the tile is staged, all at
  // once: read row by row inside the store loop, each wave would wait sixteen times.
  constexpr int kRowsPerWave = kBT / 4;
  float xv[(LOG || PREP) ? kRowsPerWave : 1][(LOG || PREP) ? NQ : 1];
  if (LOG || PREP) {
#pragma unroll
    for (int rr = 0; rr < kRowsPerWave; ++rr)
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const int x = x0 + wave + 4 * rr, k = lane + 64 * q;
        xv[rr][q] = (x < n && k < Wx) ? xo[(long)x * Wx + k] : 0.f;
      }
  }
  __syncthreads();
  float* ct = sl;  // [64][ld_own]
#pragma unroll
  for (int q = 0; q < kMaxKB; ++q) {
    const int k0 = 8 * (wave + 4 * q);
    if (k0 >= Wx) break;
#pragma unroll
    for (int t = 0; t < 8; ++t)
      if (k0 + t < Wx)
        ct[lane * ld_own + k0 + t] = acc[q][t];
  }
  __syncthreads();
#pragma unroll
  for (int rr = 0; rr < kRowsPerWave; ++rr) {
    const int r = wave + 4 * rr, x = x0 + r;
    if (x >= n) break;
    if ((LOG || PREP) && badrow[r]) {  // recompute this row cell by cell from memory
      for (int k = lane; k < Wx; k += 64) {
        if (GRAD_A) band_bwd_a_cell<GENBMM_BAND_LOG>(p, bn + x, x, k);
        else band_bwd_b_cell<GENBMM_BAND_LOG>(p, bn + x, x, k);
      }
    } else if (LOG) {
      const float sh = sh_own[r] == -INFINITY ? 0.f : sh_own[r];
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const int k = lane + 64 * q;
        if (k >= Wx) break;
        // exp(x - shift); cells outside the matrix are excluded from the row maximum
        // and their sum is 0
        const float acv = ct[r * ld_own + k];
        gradb[(long)x * Wx + k] = to_elem<elem_t>(acv == 0.f ? 0.f : fast_exp2((xv[rr][q] - sh) * kLog2e) * acv);
      }
    } else if (PREP) {
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const int k = lane + 64 * q;
        if (k < Wx) gradb[(long)x * Wx + k] = to_elem<elem_t>(xv[rr][q] * ct[r * ld_own + k]);
      }
    } else {
      for (int k = lane; k < Wx; k += 64) gradb[(long)x * Wx + k] = to_elem<elem_t>(ct[r * ld_own + k]);
    }
  }
}

inline int bwd_sl_floats(const StripDims& d) { return max(kBR * d.ld_sl, kBT * d.ld_own); }
inline size_t bwd_strip_bytes(const StripDims& d, bool log_mode) {
  (void)log_mode;
  return sizeof(float) * ((size_t)bwd_sl_floats(d) + (size_t)kBR * kBC + kBT + kBR + kBT);
}

inline StripDims strip_dims(int w_own, int w_sl) {
  StripDims d;
  d.ld_own = odd(w_own);
  d.ld_sl = odd(w_sl + 2 * kBP);
  d.bytes = sizeof(float) * ((size_t)kBT * d.ld_own + (size_t)kBR * d.ld_sl + kBT + kBR);
  return d;
}

}  // namespace GENBMM_NS
