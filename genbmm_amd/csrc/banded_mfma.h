// Banded (+,*) products on the matrix cores: forward, grad_a and grad_b of the
// plain product, and of the log product on the forward's workspace (operands
// exp(a - alpha), exp(b - beta), see banded_strip.h), as one kernel template.
//
// In dense coordinates all three are products C[x, y] = sum_z P(x, z) * Q(z, y)
// whose operands are rows of band tensors read with a skew:
//   forward   x = i, y = o, z = m :  a[i][m - i + lu_a]   * b[o][m - o + lu_b]    -> out[i][o - i + lu_o]
//   grad_a    x = i, y = m, z = o :  g'[i][o - i + lu_o]  * b[o][m - o + lu_b]    -> ga[i][m - i + lu_a]
//   grad_b    x = o, y = m, z = i :  g'[i][o - i + lu_o]  * a[i][m - i + lu_a]    -> gb[o][m - o + lu_b]
// (m = i + k - lu_a is the dense row that a[i][k] and b[o][k2] share; x, y and z all
// lie in [0, n).)  A workgroup owns a strip of consecutive rows x - 64 in the forward,
// 32 in the gradients, whose first operand is twice as wide.  The rows of both
// operands that the strip meets are copied to LDS as they lie in memory, one
// contiguous block each, in 16-byte pieces.  The result is cut into 16 x 16 tiles of
// (x, y); a tile's sum runs over the z that any of its cells can meet, in steps of 4,
// the depth of v_mfma_f32_16x16x4_f32.  Every lane reads one value of P and one of Q
// per instruction, from an address that is affine in z; a lane whose (x, z) or (z, y)
// is outside its band or outside the matrix feeds zero instead.  Only the first and
// last steps of a tile need that test: in the steps between, every lane is inside.
// About two thirds of the multiply-adds issued are inside the band for 65
// diagonals; the matrix cores still finish them several times faster than the vector
// pipes finish the exact count, because on the vector pipes every multiply-add of this
// product needs an LDS read of its own.
//
// Forward: one wave per 16-row tile row.  Gradients: two waves per tile row, the
// steps dealt to them in two equal runs, a tile cut by the boundary being summed from
// both (first wave stores, second adds).  The result goes through LDS so that the
// strip's rows are written as one contiguous run.
//
// Values that are not finite cannot take this road (0 * inf for a lane that is outside
// while its partner is inside): a strip that stages one is recomputed cell by cell
// by the per-cell routines, and in the log backward a row fed by an unusable
// H = g / S is (as in the strip kernels).
#pragma once

#include <cfloat>
#include <cstdint>

#include "banded_strip.h"

namespace genbmm {

constexpr int kMmTiles = 12;   // 16-column tiles per tile row, at most (result width <= 177)
constexpr int kMmFwd = 0, kMmGradA = 1, kMmGradB = 2;
constexpr int kMmSlack = 8;    // spare floats around a staged block
typedef float mm_f4 __attribute__((ext_vector_type(4)));

inline constexpr int mm_rows(int kind) { return kind == kMmFwd ? 64 : 32; }

struct MmDims {
  int pp, qp;       // row stride of P / Q in LDS
  int q_off;        // float offset of Q's block (P's is kMmSlack)
  int ops_floats;   // floats of both operand blocks
  int q_rows;       // rows of Q the strip meets
  size_t bytes;
};

inline MmDims mm_dims(int kind, int Wa, int Wb, int Wo) {
  MmDims d;
  const int rows = mm_rows(kind);
  const int wout = kind == kMmFwd ? Wo : kind == kMmGradA ? Wa : Wb;
  const int wp = kind == kMmFwd ? Wa : Wo, wq = kind == kMmGradB ? Wa : Wb;
  d.q_rows = rows + Wo - 1 + (kind == kMmFwd ? 0 : 3);
  // The 16 rows that one instruction reads lie (row stride - 1) apart once the skew is
  // taken off (+ 1 for the g' tile of grad_b, walked against z): twice an odd number
  // spreads them over all banks.  Rows addressed along z, 4 per instruction and 16
  // consecutive cells of each: 16 banks apart.
  d.pp = wp;
  while ((d.pp & 3) != (kind == kMmGradB ? 1 : 3)) ++d.pp;
  d.qp = wq;
  if (kind == kMmFwd) {
    while ((d.qp & 3) != 3) ++d.qp;
  } else {
    while (((d.qp - 1) & 31) != 16) ++d.qp;
  }
  // a block: up to 3 cells before the first wanted one and one row gap, the rows, and
  // the cells that the last piece carries past the end (one more gap on)
  d.q_off = (kMmSlack + rows * d.pp + 2 * (d.pp - wp) + kMmSlack + 3) & ~3;
  d.ops_floats = (d.q_off + d.q_rows * d.qp + 2 * (d.qp - wq) + kMmSlack + 3) & ~3;
  const int tile = max(d.ops_floats, rows * wout);
  // operands | result tile, alpha [rows], beta [q_rows], flags [rows + 4]
  d.bytes = sizeof(float) * ((size_t)tile + rows + d.q_rows + rows + 4);
  return d;
}
inline bool mm_tiles_ok(int Wa, int Wb, int Wo) {
  (void)Wa;
  (void)Wb;
  return (Wo + 30) / 16 <= kMmTiles;
}

// `count` floats starting at tensor[first] - rows of W floats - read in 16-byte pieces
// from the aligned address below and laid down with row stride `pitch`:
// tensor[first + r * W + k] lands at L[origin() + r * pitch + k].
// load() only issues the reads of one batch of 256 * U pieces, store() consumes them.
template <int U>
struct MmFlat {
  mm_f4 v[U];
  int nvec, lead, W, gap;
  unsigned magic;  // ceil(2^32 / W)
  const float* abeg;
  bool inside;     // every piece lies inside the tensor

  // [tensor, tensor_end): the whole tensor; a piece that crosses its ends is read float by float
  __device__ __forceinline__ void init(const float* tensor, const float* tensor_end, long first, int count,
                                       int W_, int pitch) {
    const float* beg = tensor + first;
    lead = (int)((reinterpret_cast<uintptr_t>(beg) & 15) >> 2);
    abeg = beg - lead;
    nvec = count > 0 ? (lead + count + 3) >> 2 : 0;
    W = W_;
    gap = pitch - W_;
    magic = (unsigned)((0x100000000ull + (unsigned)W - 1) / (unsigned)W);
    inside = abeg >= tensor && abeg + 4 * (long)nvec <= tensor_end;
  }
  __device__ __forceinline__ int origin() const { return lead + gap; }
  __device__ __forceinline__ bool more(int batch) const { return batch * 256 * U < nvec; }
  __device__ __forceinline__ void load(const float* lo, const float* hi, int batch, int tid) {
    if (inside) {  // uniform
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int vi = tid + 256 * (u + batch * U);
        v[u] = mm_f4{0.f, 0.f, 0.f, 0.f};
        if (vi < nvec) v[u] = *reinterpret_cast<const mm_f4*>(abeg + 4 * vi);
      }
      return;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int vi = tid + 256 * (u + batch * U);
      mm_f4 x = mm_f4{0.f, 0.f, 0.f, 0.f};
      if (vi < nvec) {
        const float* q = abeg + 4 * vi;
        for (int t = 0; t < 4; ++t)
          if (q + t >= lo && q + t < hi) x[t] = q[t];
      }
      v[u] = x;
    }
  }
  // returns whether this thread saw a value that is not finite.  Piece v holds the flat
  // cells 4 v - lead ...; with u = 4 v + W - lead, its first cell is in row u / W - 1
  // (row -1: the cells before the first wanted one), and W >= 4 lets it cross into one
  // more row at most.
  __device__ __forceinline__ bool store(float* __restrict__ L, int batch, int tid) const {
    bool bad = false;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int vi = tid + 256 * (u + batch * U);
      if (vi < nvec) {
        const mm_f4 x = v[u];
        bad |= !(fabsf(x[0]) <= FLT_MAX) || !(fabsf(x[1]) <= FLT_MAX) || !(fabsf(x[2]) <= FLT_MAX) ||
               !(fabsf(x[3]) <= FLT_MAX);
        const int f = 4 * vi, uu = f + W - lead;
        const int r1 = (int)__umulhi((unsigned)uu, magic), k = uu - r1 * W;
        float* at = L + (f + r1 * gap);
        const int nb = W - k;  // cells of the piece before its row ends, at least one
        at[0] = x[0];
#pragma unroll
        for (int t = 1; t < 4; ++t) at[t + (t >= nb ? gap : 0)] = x[t];
      }
    }
    return bad;
  }
  // v = g, rs.v = R = 1/S of the same cells (read with the same lead): v becomes
  // H = g * R, NaN where R < 0 (the cell was computed exactly, its 1/S is not usable), and
  // this strip's cells of it go to `h`, laid out like g - the other gradient reads them
  // there.  h_vec: h + (abeg - tensor) is 16-byte aligned and every piece lies inside.
  __device__ __forceinline__ void make_h(const MmFlat& rs, float* __restrict__ h, const float* tensor,
                                         bool h_vec, int count, int batch, int tid) {
    float* hb = h + (abeg - tensor);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int vi = tid + 256 * (u + batch * U);
      if (vi < nvec) {
        mm_f4 x = v[u];
        const mm_f4 r = rs.v[u];
#pragma unroll
        for (int t = 0; t < 4; ++t) x[t] = r[t] < 0.f ? __builtin_nanf("") : x[t] * r[t];
        v[u] = x;
        if (h_vec) {
          *reinterpret_cast<mm_f4*>(hb + 4 * vi) = x;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int e = 4 * vi + t - lead;
            if (e >= 0 && e < count) hb[4 * vi + t] = x[t];
          }
        }
      }
    }
  }
  // the rows (first one row_first) that hold a value that is not finite
  __device__ __forceinline__ void flag_rows(int batch, int tid, int count, int row_first, int* flags) const {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int vi = tid + 256 * (u + batch * U);
      if (vi < nvec) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int e = 4 * vi + t - lead;
          if (e >= 0 && e < count && !(fabsf(v[u][t]) <= FLT_MAX)) flags[row_first + e / W] = 1;
        }
      }
    }
  }
};

// g' for grad_b: T[c * pitch + j] = g'[i][j] with i = x0 + c - j + lu_o, for the 32
// rows o = x0 + c of the strip (zero where g' has no such cell); read as runs of 32
// cells along the rows of g'.
template <bool ROWFLAG, int U>
struct MmSkew {
  float v[U];
  int total;

  __device__ __forceinline__ void init(int Wo) { total = (Wo + 31) * 32; }
  __device__ __forceinline__ bool more(int batch) const { return batch * 256 * U < total; }
  // Cell number tid + 256 u is (row r of g' counted from ilo, column c of the strip) with
  // c = tid % 32 fixed and r = tid / 32 + 8 u: its address moves by 8 (Wo - 1) floats per
  // u, its band index j = c + Wo - 1 - r by -8.  j is inside the band for r in
  // [c, c + Wo); the cell exists for the r that are also rows of the matrix.
  __device__ __forceinline__ void load(const float* __restrict__ src, int Wo, int r_lu, int n, int x0,
                                       int batch, int tid) {
    const int ilo = x0 + r_lu - (Wo - 1), c = tid & 31, r0 = (tid >> 5) + 8 * U * batch;
    const int rlo = max(c, -ilo), rhi = x0 + c < n ? min(c + Wo, n - ilo) : rlo;
    const float* q = src + ((long)(ilo + r0) * Wo + (c + Wo - 1 - r0));
    const long step = 8L * (Wo - 1);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = r0 + 8 * u;
      v[u] = (r >= rlo && r < rhi) ? q[u * step] : 0.f;
    }
  }
  __device__ __forceinline__ void store(float* __restrict__ T, int pitch, int Wo, int batch, int tid,
                                        int* flags) const {
    const int c = tid & 31, r0 = (tid >> 5) + 8 * U * batch;
    float* t = T + c * pitch + (c + Wo - 1 - r0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = r0 + 8 * u;
      if (r >= c && r < c + Wo) {
        const float x = v[u];
        if (!(fabsf(x) <= FLT_MAX)) flags[ROWFLAG ? c : 0] = 1;
        t[-8 * u] = x;
      }
    }
  }
};

__device__ __forceinline__ int mm_clamp(int x, int lo, int hi) { return min(max(x, lo), hi); }

// The exact recompute of one cell, inline: a call would give the kernel a stack frame
// that every lane writes to memory (168 bytes each, 168 MiB per launch at 64 x 4096).
__device__ __forceinline__ float mm_fwd_cell_log_exact(const BandArgs& p, long bi, int i, int j) {
  band_fwd_cell<GENBMM_BAND_LOG>(p, bi, i, j);
  return p.o0[bi * p.Wo + j];
}

template <int KIND, bool PREP>
__global__ __launch_bounds__(256, 2) void k_band_mm(const BandArgs p, int strips, const MmDims d, long cells_a,
                                                    long cells_b, long cells_o, int fuse_h) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  constexpr bool FWD = KIND == kMmFwd, GA = KIND == kMmGradA, GB = KIND == kMmGradB;
  constexpr int ROWS = FWD ? 64 : 32;   // result rows per workgroup
  constexpr int SPLIT = FWD ? 1 : 2;    // waves per 16-row tile row
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wg = xcd_strip_id();
  const int batch = wg / strips, x0 = (wg - batch * strips) * ROWS;
  const int n = p.n, Wa = p.Wa, Wb = p.Wb, Wo = p.Wo, r_lu = p.r_lu;
  const int a_ld = Wa - 1 - p.a_lu, b_ld = Wb - 1 - p.b_lu;
  const long bn = (long)batch * n;
  const int Wq = GB ? Wa : Wb, luq = GB ? p.a_lu : p.b_lu;
  const int Wp = FWD ? Wa : Wo;
  const int Wout = FWD ? Wo : GA ? Wa : Wb;
  float* PL = smem + kMmSlack;   // P block: 16-byte pieces from here
  float* QL = smem + d.q_off;
  float* S = smem;               // result tile [ROWS][Wout], in place of the operands
  const int tile_floats = max(d.ops_floats, ROWS * Wout);
  float* al = smem + tile_floats;            // [ROWS]    forward of the log product
  float* be = al + ROWS;                     // [q_rows]
  int* badrow = reinterpret_cast<int*>(be + d.q_rows);  // [ROWS] rows to redo, then: the whole strip
  int* redo = badrow + ROWS;

  // ---- staging: rows of Q from q0 on, rows of P from x0 on, as far as they exist
  const int q0 = GB ? x0 + r_lu - (Wo - 1) : x0 - r_lu;
  const float* at = PREP ? p.ws_ea : p.a;
  const float* bt = PREP ? p.ws_eb : p.b;
  const float* gt = FWD ? nullptr : (PREP ? p.ws_h : p.g);
  const float* qt = GB ? at : bt;
  const long cells_q = GB ? cells_a : cells_b;
  const int qr0 = max(q0, 0), qr1 = min(q0 + d.q_rows, n);  // existing rows of Q
  const int pr1 = min(x0 + ROWS, n);
  MmFlat<14> sq;
  MmFlat<6> sp, sr;
  MmSkew<PREP, 20> sk;
  // grad_a of the prepared log product can form H = g / S itself while it stages it, and
  // leave it in the workspace for grad_b (fuse_h: g, 1/S and H start on the same 16-byte phase)
  const bool mk_h = GA && PREP && fuse_h != 0;
  const float* pt = FWD ? at : (mk_h ? p.g : gt);
  sq.init(qt, qt + cells_q, (bn + qr0) * Wq, (qr1 - qr0) * Wq, Wq, d.qp);
  sq.load(qt, qt + cells_q, 0, tid);
  if (GB) {
    sk.init(Wo);
    sk.load(gt + bn * Wo, Wo, r_lu, n, x0, 0, tid);
  } else {
    sp.init(pt, pt + (FWD ? cells_a : cells_o), (bn + x0) * Wp, (pr1 - x0) * Wp, Wp, d.pp);
    sp.load(pt, pt + (FWD ? cells_a : cells_o), 0, tid);
    if (mk_h) {
      sr.init(p.ws_r, p.ws_r + cells_o, (bn + x0) * Wp, (pr1 - x0) * Wp, Wp, d.pp);
      sr.load(p.ws_r, p.ws_r + cells_o, 0, tid);
    }
  }
  // forward of the log product: the row maxima too are requested before anything is waited for
  float alv = 0.f, bev = 0.f;
  if (FWD && PREP) {
    if (tid < ROWS && x0 + tid < n) alv = p.ws_al[bn + x0 + tid];
    const int o = q0 + tid;
    if (tid < d.q_rows && o >= 0 && o < n) bev = p.ws_be[bn + o];
  }
  if (tid <= ROWS) badrow[tid] = 0;
  __syncthreads();
  bool bad = sq.store(QL, 0, tid);
  for (int b = 1; sq.more(b); ++b) {
    sq.load(qt, qt + cells_q, b, tid);
    bad |= sq.store(QL, b, tid);
  }
  if (GB) {
    int* pflags = PREP ? badrow : redo;
    sk.store(PL, d.pp, Wo, 0, tid, pflags);
    for (int b = 1; sk.more(b); ++b) {
      sk.load(gt + bn * Wo, Wo, r_lu, n, x0, b, tid);
      sk.store(PL, d.pp, Wo, b, tid, pflags);
    }
  } else {
    for (int b = 0; b == 0 || sp.more(b); ++b) {
      if (b > 0) {
        sp.load(pt, pt + (FWD ? cells_a : cells_o), b, tid);
        if (mk_h) sr.load(p.ws_r, p.ws_r + cells_o, b, tid);
      }
      if (mk_h) sp.make_h(sr, p.ws_h, pt, sp.inside, (pr1 - x0) * Wp, b, tid);
      const bool pbad = sp.store(PL, b, tid);
      if (PREP && GA) {
        if (pbad) sp.flag_rows(b, tid, (pr1 - x0) * Wp, 0, badrow);
      } else {
        bad |= pbad;
      }
    }
  }
  if (bad) *redo = 1;
  if (FWD && PREP) {
    if (tid < ROWS) al[tid] = alv;
    if (tid < d.q_rows) be[tid] = bev;
    for (int t = tid + 256; t < d.q_rows; t += 256) {
      const int o = q0 + t;
      be[t] = (o >= 0 && o < n) ? p.ws_be[bn + o] : 0.f;
    }
  }
  __syncthreads();
  // element (row, k) of P / Q, rows counted from x0 / q0
  const int pp = d.pp, qp = d.qp;
  const float* Pt = GB ? PL : PL + sp.origin();
  const float* Qt = QL + sq.origin() - (qr0 - q0) * qp;

  // ---- tiles
  const int xt = wave / SPLIT, part = wave % SPLIT;
  const int x0t = x0 + 16 * xt;
  const int l15 = lane & 15, zq = lane >> 4;
  // y of tile ty starts at x0t + cy + 16 ty; z runs over
  // [max(x0t + c1, y0t + c2, 0), min(x0t + 15 + c3, y0t + 15 + c4, n - 1)]; result column y - x - cy
  const int cy = FWD ? -r_lu : GA ? -p.a_lu : -p.b_lu;
  const int c1 = FWD ? -p.a_lu : GA ? -r_lu : r_lu - (Wo - 1);
  const int c2 = FWD ? -p.b_lu : GA ? -b_ld : -a_ld;
  const int c3 = FWD ? a_ld : GA ? Wo - 1 - r_lu : r_lu;
  const int c4 = FWD ? b_ld : GA ? p.b_lu : p.a_lu;
  const int ny = (Wout + 30) >> 4;
  int total = 0;
  for (int ty = 0; SPLIT > 1 && ty < ny; ++ty) {
    const int y0t = x0t + cy + 16 * ty;
    const int zlo = max(max(x0t + c1, y0t + c2), 0), zhi = min(min(x0t + 15 + c3, y0t + 15 + c4), n - 1);
    total += zhi >= zlo ? (zhi - zlo + 4) >> 2 : 0;
  }
  const int lo = SPLIT == 1 ? 0 : part ? (total + 1) >> 1 : 0;
  const int hi = SPLIT == 1 ? 0x3fffffff : part ? total : (total + 1) >> 1;

  // this lane's row of P: the z inside are [plo, plo + pspan]
  constexpr int kNone = 0x3fffffff;
  const int x = x0t + l15;
  int plo = max(x + c1, 0), pspan = min(x + c3, n - 1) - plo;
  if (x >= n || pspan < 0) {
    plo = kNone;
    pspan = 0;
  }
  // P(x, z) = Pt[pbase + psign * z]
  constexpr int psign = GB ? -1 : 1;
  const int prow = (16 * xt + l15) * pp;
  const int pbase = GB ? prow + x + r_lu : prow - x + (FWD ? p.a_lu : r_lu);
  const int dq = FWD ? 4 : 4 * (qp - 1);

  mm_f4 acc[kMmTiles];
  unsigned mine = 0;
  int base = 0;
#pragma unroll
  for (int ty = 0; ty < kMmTiles; ++ty) {
    acc[ty] = mm_f4{0.f, 0.f, 0.f, 0.f};
    if (ty < ny) {
      const int y0t = x0t + cy + 16 * ty;
      const int zlo = max(max(x0t + c1, y0t + c2), 0), zhi = min(min(x0t + 15 + c3, y0t + 15 + c4), n - 1);
      const int nst = zhi >= zlo ? (zhi - zlo + 4) >> 2 : 0;
      const int s0 = max(lo - base, 0), s1 = min(hi - base, nst);
      base += nst;
      if (s0 < s1) {
        mine |= 1u << ty;
        // steps in which every lane of the tile is inside both bands and the matrix
        const int zc0 = max(max(x0t + 15 + c1, y0t + 15 + c2), 0);
        const int zc1 = min(min(x0t + c3, y0t + c4), n - 1);
        const bool rows_in = x0t + 15 < n && y0t >= 0 && y0t + 15 < (FWD ? qr1 : n);
        int sc0 = (zc0 - zlo + 3) >> 2, sc1 = zc1 - 3 >= zlo ? ((zc1 - 3 - zlo) >> 2) + 1 : 0;
        if (!rows_in || sc1 < sc0) sc0 = sc1 = s0;
        sc0 = mm_clamp(sc0, s0, s1);
        sc1 = mm_clamp(sc1, sc0, s1);
        // this lane's column of Q
        const int y = y0t + l15;
        int qlo = max(y + c2, 0), qspan = min(y + c4, n - 1) - qlo;
        if (y < 0 || y >= n || qspan < 0) {
          qlo = kNone;
          qspan = 0;
        }
        // forward: Qt[(y - q0) * qp + z - y + lu_b]; gradients: Qt[(z - q0) * qp + y - z + lu]
        const int qbase = FWD ? (y - q0) * qp - y + luq : y + luq - q0 * qp;
        const int qz = FWD ? 1 : qp - 1;
        mm_f4 c = acc[ty];
        // One walk through the tile's steps: first steps with the test, the steps in
        // which every lane is inside without it, last steps with it again.  A lane outside
        // feeds zero; what it reads instead (possibly beyond the staged rows, LDS has no
        // faults) does not matter.
        const int z = zlo + 4 * s0 + zq;
        const float* pa = Pt + pbase + psign * z;
        const float* pb = Qt + qbase + qz * z;
        unsigned zp = (unsigned)(z - plo), zy = (unsigned)(z - qlo);
        int s = s0;
        for (; s < sc0; ++s) {
          float a = *pa, b = *pb;
          a = zp <= (unsigned)pspan ? a : 0.f;
          b = zy <= (unsigned)qspan ? b : 0.f;
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
          pa += 4 * psign;
          pb += dq;
          zp += 4;
          zy += 4;
        }
        zp += 4 * (sc1 - sc0);
        zy += 4 * (sc1 - sc0);
        for (; s + 4 <= sc1; s += 4) {
          const float a0 = pa[0], a1 = pa[4 * psign], a2 = pa[8 * psign], a3 = pa[12 * psign];
          const float b0 = pb[0], b1 = pb[dq], b2 = pb[2 * dq], b3 = pb[3 * dq];
          pa += 16 * psign;
          pb += 4 * dq;
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, b0, c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, b1, c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a2, b2, c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a3, b3, c, 0, 0, 0);
        }
        for (; s < sc1; ++s) {
          const float a0 = pa[0], b0 = pb[0];
          pa += 4 * psign;
          pb += dq;
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, b0, c, 0, 0, 0);
        }
        for (; s < s1; ++s) {
          float a = *pa, b = *pb;
          a = zp <= (unsigned)pspan ? a : 0.f;
          b = zy <= (unsigned)qspan ? b : 0.f;
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
          pa += 4 * psign;
          pb += dq;
          zp += 4;
          zy += 4;
        }
        acc[ty] = c;
      }
    }
  }
  __syncthreads();  // the operands are consumed: their place becomes the result tile

  // lane holds rows 4 zq + r, column l15 of each of its tiles; result column 16 ty + l15 - row
  int srow[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) srow[r] = (16 * xt + 4 * zq + r) * Wout + l15 - (4 * zq + r);
#pragma unroll
  for (int phase = 0; phase < SPLIT; ++phase) {
    if (part == phase) {
#pragma unroll
      for (int ty = 0; ty < kMmTiles; ++ty) {
        if (ty < ny && (phase == 0 || ((mine >> ty) & 1u))) {
          const bool inner = 16 * ty - 15 >= 0 && 16 * ty + 15 < Wout;  // no lane of the tile is outside
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int col = 16 * ty + l15 - (4 * zq + r);
            if (inner || (col >= 0 && col < Wout)) {
              float* sc = S + srow[r] + 16 * ty;
              *sc = phase == 0 ? acc[ty][r] : *sc + acc[ty][r];
            }
          }
        }
      }
    }
    __syncthreads();
  }

  // ---- rows out: one contiguous run of memory
  const int rows = min(ROWS, n - x0);
  const int cells = rows * Wout;
  const bool whole = *redo != 0;
  float* ob = (GB ? p.o1 : p.o0) + (bn + x0) * Wout;
  if (!PREP && !whole) {
    if ((reinterpret_cast<uintptr_t>(ob) & 15) == 0) {
      for (int e = 4 * tid; e < cells; e += 1024) {
        if (e + 3 < cells) {
          *reinterpret_cast<mm_f4*>(ob + e) = *reinterpret_cast<const mm_f4*>(S + e);
        } else {
          for (int t = e; t < cells; ++t) ob[t] = S[t];
        }
      }
    } else {
      for (int e = tid; e < cells; e += 256) ob[e] = S[e];
    }
    return;
  }
  const unsigned magic = (unsigned)((0x100000000ull + (unsigned)Wout - 1) / (unsigned)Wout);
  const float thr = fast_exp2(-kBandGuardBits);
  const float* xe = PREP && !FWD ? (GA ? p.ws_ea : p.ws_eb) + (bn + x0) * Wout : nullptr;
  float* rb = PREP && FWD ? p.ws_r + (bn + x0) * Wout : nullptr;
  // Prepared log product away from trouble: four cells per lane, 16-byte loads and stores
  // (a quarter of the index arithmetic and memory instructions of the cell-by-cell loop).
  const bool vec_ok = PREP && !whole && (cells & 3) == 0 && Wout >= 4 && (reinterpret_cast<uintptr_t>(ob) & 15) == 0 &&
                      (FWD ? (reinterpret_cast<uintptr_t>(rb) & 15) == 0 : (reinterpret_cast<uintptr_t>(xe) & 15) == 0);
  if (PREP && vec_ok) {
    for (int e = 4 * tid; e < cells; e += 1024) {
      const mm_f4 sv = *reinterpret_cast<const mm_f4*>(S + e);
      const int r0 = (int)__umulhi((unsigned)e, magic), k0 = e - r0 * Wout;
      mm_f4 ov, rv4;
      bool redo_cell[4];
      if (FWD) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const bool wrap = k0 + t >= Wout;  // Wout >= 4: one row change at most
          const int r = r0 + (wrap ? 1 : 0), k = k0 + t - (wrap ? Wout : 0);
          const int o = x0 + r + k - r_lu;
          float v = sv[t], rv = 0.f;
          redo_cell[t] = false;
          if (o >= 0 && o < n) {
            const float sh = al[r] + be[o - q0];
            if ((v >= thr) && (v < INFINITY) && (sh > 0.9f * kFloor) && (sh < INFINITY)) {
              rv = __builtin_amdgcn_rcpf(v);
              v = __builtin_fmaf(fast_log2(v), kLn2, sh);
            } else {
              redo_cell[t] = true;
              rv = -1.f;  // tells the backward that 1/S is not usable here
            }
          } else {
            v = 0.f;  // outside the matrix: the reference's zero fill
          }
          ov[t] = v;
          rv4[t] = rv;
        }
        // factoring not exact for a cell: recompute it from memory
#pragma unroll
        for (int t = 0; t < 4; ++t)
          if (redo_cell[t]) {
            const bool wrap = k0 + t >= Wout;
            const int r = r0 + (wrap ? 1 : 0), k = k0 + t - (wrap ? Wout : 0);
            ov[t] = mm_fwd_cell_log_exact(p, bn + x0 + r, x0 + r, k);
          }
        *reinterpret_cast<mm_f4*>(ob + e) = ov;
        *reinterpret_cast<mm_f4*>(rb + e) = rv4;
      } else {
        const mm_f4 xv = *reinterpret_cast<const mm_f4*>(xe + e);
        const bool wrapped = k0 + 3 >= Wout;
        if (!badrow[r0] && !(wrapped && badrow[r0 + 1])) {
          *reinterpret_cast<mm_f4*>(ob + e) = xv * sv;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const bool wrap = k0 + t >= Wout;
            const int r = r0 + (wrap ? 1 : 0), k = k0 + t - (wrap ? Wout : 0);
            if (badrow[r]) {
              if (GA) band_bwd_a_cell<GENBMM_BAND_LOG>(p, bn + x0 + r, x0 + r, k);
              else band_bwd_b_cell<GENBMM_BAND_LOG>(p, bn + x0 + r, x0 + r, k);
            } else {
              ob[e + t] = xv[t] * sv[t];
            }
          }
        }
      }
    }
    return;
  }
  for (int e = tid; e < cells; e += 256) {
    float v = S[e];
    const int r = Wout == 1 ? e : (int)__umulhi((unsigned)e, magic), k = e - r * Wout;
    const int xx = x0 + r;
    if (FWD && PREP) {
      const int o = xx + k - r_lu;
      float rv = 0.f;
      if (o >= 0 && o < n) {
        const float sh = al[r] + be[o - q0];
        if (!whole && (v >= thr) && (v < INFINITY) && (sh > 0.9f * kFloor) && (sh < INFINITY)) {
          rv = __builtin_amdgcn_rcpf(v);
          v = __builtin_fmaf(fast_log2(v), kLn2, sh);
        } else {  // factoring not exact for this cell: recompute it from memory
          v = mm_fwd_cell_log_exact(p, bn + xx, xx, k);
          rv = -1.f;  // tells the backward that 1/S is not usable here
        }
      } else {
        v = 0.f;  // outside the matrix: the reference's zero fill
      }
      ob[e] = v;
      rb[e] = rv;
    } else if (FWD) {
      band_fwd_cell<GENBMM_BAND_MUL>(p, bn + xx, xx, k);
    } else if (PREP) {
      if (whole || badrow[r]) {
        if (GA) band_bwd_a_cell<GENBMM_BAND_LOG>(p, bn + xx, xx, k);
        else band_bwd_b_cell<GENBMM_BAND_LOG>(p, bn + xx, xx, k);
      } else {
        ob[e] = xe[e] * v;
      }
    } else {
      if (GA) band_bwd_a_cell<GENBMM_BAND_MUL>(p, bn + xx, xx, k);
      else band_bwd_b_cell<GENBMM_BAND_MUL>(p, bn + xx, xx, k);
    }
  }
}

}  // namespace genbmm
