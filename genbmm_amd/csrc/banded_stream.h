// Banded (+,*) products on the matrix cores as streams: forward and grad_a of the plain
// product and of the log product on the forward's workspace.
//
// Same arithmetic as banded_mfma.h - in dense coordinates C[x, y] = sum_z P(x, z) Q(z, y)
// cut into 16 x 16 tiles for v_mfma_f32_16x16x4_f32 - but a workgroup does not own one
// strip: it walks down a run of rows, 64 at a time, and keeps in LDS the window of the
// second operand's rows that the current 64 rows meet (64 + Wo - 1 of them).  From block
// to block the window moves down by 64 rows inside LDS and only 64 new rows are read from
// memory, while the previous block's tiles are being computed (the reads wait in
// registers).  Every operand row therefore crosses from memory to LDS once per run instead
// of once per strip (three to five times at 65 diagonals), which is what bounded the
// strip kernels.
//
// Staged rows lie kGap cells apart and the cells between them hold zeros, as do the cells
// of a row that fall outside the matrix and the rows beyond its ends.  A tile's steps can
// then run over the union of its 16 rows' ranges without any test: a lane that is outside
// its band reads a zero.  The window always starts at the same place, so what a lane needs
// to know about a tile - where its operands start, how many steps - is computed once per
// launch, not per block.
//
// A value that is not finite cannot take this road (0 * inf): whichever result cell it
// reaches comes out as NaN or inf and is recomputed from memory by the per-cell routine
// when the block's results are written.
#pragma once

#include <cfloat>

#include "banded_mfma.h"

namespace genbmm {

// Result rows per block: 64 (eight waves: four tile rows x two halves of the tiles) or 32
// (four waves), whichever lets two workgroups share a compute unit's LDS - one's tiles
// then run while the other stages and writes.  Eight threads per row either way.
constexpr int kSGap = 18;         // a lane reads up to 15 + 3 cells beside its own band
constexpr int kSTiles = 6;        // tiles per wave, at most (result width <= 162)
constexpr int kSLead = 24;        // zero cells in front of a block of rows
constexpr int kSUQ = 3;           // 16-byte pieces per thread: 64 rows of up to 95 cells
constexpr int kSUP = 6;           //                            64 rows of up to 191 cells
constexpr int kSShift = 16;       // pieces per thread when the window moves, at most
constexpr int kStFwd = 0, kStGradA = 1;

struct StreamDims {
  int pp, qp;       // row pitch of P / Q in LDS
  int qr;           // rows of the Q window
  int p_off, q_off, s_off, al_off, be_off, total;  // float offsets
  size_t bytes;
};

inline StreamDims stream_dims(int kind, int rows, int Wa, int Wb, int Wo) {
  StreamDims d;
  const int kSRows = rows;
  const int wp = kind == kStFwd ? Wa : Wo, wq = Wb, wout = kind == kStFwd ? Wo : Wa;
  // 16 rows read by one instruction lie (pitch - 1) apart: twice an odd number spreads
  // them over all banks
  d.pp = wp + kSGap;
  while ((d.pp & 3) != 3) ++d.pp;
  d.qp = wq + kSGap;
  while ((d.qp & 3) != 3) ++d.qp;
  d.qr = kSRows + Wo - 1;
  d.p_off = kSLead;
  d.q_off = (d.p_off + kSRows * d.pp + kSLead + 3) & ~3;
  // grad_a: 4 rows more, the last step of a tile reads past the window
  d.s_off = (d.q_off + (d.qr + (kind == kStFwd ? 0 : 4)) * d.qp + 3) & ~3;
  d.al_off = (d.s_off + kSRows * wout + 3) & ~3;
  d.be_off = d.al_off + kSRows;
  d.total = d.be_off + ((d.qr + 3) & ~3);
  d.bytes = sizeof(float) * (size_t)d.total;
  return d;
}

// Rows [row_lo, row_lo + nrows) of one batch item's (n x W) band tensor, on their way
// from memory to LDS: load() issues the reads (16-byte pieces from the aligned address
// below the first wanted cell), store() lays the rows down `pitch` apart.  Rows outside
// [0, n) and cells of a row whose dense row c + k - lu is outside [0, n) become zeros.
template <int U, int kSThreads>
struct StreamRows {
  mm_f4 v[U];
  int lead, nvec, count, e0, e1, W;
  unsigned magic;

  // item: first cell of the batch item; [tensor, tensor_end): the whole tensor
  __device__ __forceinline__ void load(const float* __restrict__ item, const float* tensor,
                                       const float* tensor_end, int row_lo, int nrows, int n, int W_,
                                       int tid) {
    W = W_;
    e0 = max(row_lo, 0) - row_lo;
    e1 = min(row_lo + nrows, n) - row_lo;
    count = e1 > e0 ? (e1 - e0) * W : 0;
    magic = (unsigned)((0x100000000ull + (unsigned)W - 1) / (unsigned)W);
    const float* beg = item + (long)(row_lo + e0) * W;
    lead = (int)((reinterpret_cast<uintptr_t>(beg) & 15) >> 2);
    const float* abeg = beg - lead;
    nvec = count > 0 ? (lead + count + 3) >> 2 : 0;
    const bool inside = abeg >= tensor && abeg + 4 * (long)nvec <= tensor_end;  // uniform
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int vi = tid + kSThreads * u;
      mm_f4 x = mm_f4{0.f, 0.f, 0.f, 0.f};
      if (vi < nvec) {
        const float* q = abeg + 4 * vi;
        if (inside) {
          x = *reinterpret_cast<const mm_f4*>(q);
        } else {
          for (int t = 0; t < 4; ++t)
            if (q + t >= tensor && q + t < tensor_end) x[t] = q[t];
        }
      }
      v[u] = x;
    }
  }

  // L: where the segment's first row (row_lo) goes.  edge: the segment may hold cells
  // outside the matrix (uniform).
  __device__ __forceinline__ void store(float* __restrict__ L, int pitch, int row_lo, int nrows, int n,
                                        int lu, int tid) const {
    const int gap = pitch - W;
    const bool edge = row_lo < lu || row_lo + nrows - 1 + (W - 1 - lu) > n - 1;
    float* L0 = L + e0 * pitch;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int vi = tid + kSThreads * u;
      if (vi < nvec) {
        const mm_f4 x = v[u];
        const int e = 4 * vi - lead;  // flat index of the piece's first cell among the wanted ones
        int r = 0, k = e;
        if (e >= 0) {
          r = (int)__umulhi((unsigned)e, magic);
          k = e - r * W;
        }
        float* at = L0 + r * pitch + k;
        const int nb = W - k;  // cells of the piece before its row ends
        if (e >= 0 && e + 3 < count && !edge) {
          at[0] = x[0];
#pragma unroll
          for (int t = 1; t < 4; ++t) at[t + (t >= nb ? gap : 0)] = x[t];
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            if (e + t >= 0 && e + t < count) {
              const bool wrap = t >= nb;
              const int c = row_lo + e0 + r + (wrap ? 1 : 0), kk = k + t - (wrap ? W : 0);
              const int m = c + kk - lu;
              at[t + (wrap ? gap : 0)] = (m >= 0 && m < n) ? x[t] : 0.f;
            }
          }
        }
      }
    }
    // rows that do not exist (beyond the ends of the matrix): zeros
    const int missing = nrows - (e1 > e0 ? e1 - e0 : 0);
    if (missing > 0) {  // uniform
      for (int c = tid; c < missing * W; c += kSThreads) {
        int r = c / W;
        const int k = c - r * W;
        if (e1 > e0 && r >= e0) r += e1 - e0;
        L[r * pitch + k] = 0.f;
      }
    }
  }
};

// One wave's tiles: ty = half, half + 2, ...  What a lane knows about each of them.
struct StreamTile {
  int pa, pb;  // float offsets of this lane's first operands of P / Q
};

template <int KIND, bool PREP, int kSRows>
__global__ __launch_bounds__(8 * kSRows, kSRows == 32 ? 2 : 1) void k_band_stream(const BandArgs p, const StreamDims d, int runs,
                                                             int run_rows, long cells_a, long cells_b,
                                                             long cells_o, int fuse_h) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  constexpr bool FWD = KIND == kStFwd;
  constexpr int kSThreads = 8 * kSRows, kTileRows = kSRows / 16;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int batch = blockIdx.x / runs;
  const int xr0 = (blockIdx.x - batch * runs) * run_rows;
  const int n = p.n, Wa = p.Wa, Wb = p.Wb, Wo = p.Wo, r_lu = p.r_lu;
  const int xr1 = min(xr0 + run_rows, n);
  const int a_ld = Wa - 1 - p.a_lu, b_ld = Wb - 1 - p.b_lu, o_ld = Wo - 1 - r_lu;
  const long bn = (long)batch * n;
  const int Wp = FWD ? Wa : Wo, Wout = FWD ? Wo : Wa;
  const int lup = FWD ? p.a_lu : r_lu;
  const int pp = d.pp, qp = d.qp, QR = d.qr;
  float* PL = smem + d.p_off;
  float* QL = smem + d.q_off;
  float* S = smem + d.s_off;
  float* al = smem + d.al_off;  // [64]  forward of the log product: row maxima of a
  float* be = smem + d.be_off;  // [QR]                              and of the window's rows of b

  // ---- operands in memory
  const float* at = PREP ? p.ws_ea : p.a;
  const float* bt = PREP ? p.ws_eb : p.b;
  // grad_a of the prepared log product can form H = g / S itself while it stages it, and
  // leave it in the workspace for grad_b (fuse_h: g, 1/S and H start on the same 16-byte phase)
  const bool mk_h = !FWD && PREP && fuse_h != 0;
  const float* pt = FWD ? at : (PREP && !mk_h ? p.ws_h : p.g);
  const long cells_p = FWD ? cells_a : cells_o;
  const float* p_item = pt + bn * Wp;
  const float* r_item = p.ws_r + bn * Wp;  // mk_h only
  const float* q_item = bt + bn * Wb;

  // ---- zeros everywhere the operands live
  for (int e = 4 * tid; e < d.s_off; e += 4 * kSThreads) *reinterpret_cast<mm_f4*>(smem + e) = mm_f4{0.f, 0.f, 0.f, 0.f};
  __syncthreads();

  // ---- tiles of this wave, once per launch
  const int xt = wave % kTileRows, half = wave / kTileRows;
  const int l15 = lane & 15, zq = lane >> 4;
  const int ny = (Wout + 30) >> 4;
  StreamTile tl[kSTiles];
  int nst[kSTiles];
  // a step moves P by 4 cells; Q by 4 cells (forward: z runs along its rows) or by 4 rows
  // and 4 cells back (grad_a: z is its row)
  const int dq = FWD ? 4 : 4 * (qp - 1);
#pragma unroll
  for (int q = 0; q < kSTiles; ++q) {
    const int ty = half + 2 * q;
    nst[q] = 0;
    tl[q].pa = tl[q].pb = 0;
    if (ty < ny) {
      // z range of the tile relative to its first row x0t: [dlo, dhi]
      int dlo, dhi;
      if (FWD) {  // y0t = x0t - lu_o + 16 ty;  z in [x - lu_a, x + ld_a] and [y - lu_b, y + ld_b]
        dlo = max(-p.a_lu, 16 * ty - r_lu - p.b_lu);
        dhi = min(15 + a_ld, 16 * ty - r_lu + 15 + b_ld);
      } else {    // y0t = x0t - lu_a + 16 ty;  z in [x - lu_o, x + ld_o] and [y - ld_b, y + lu_b]
        dlo = max(-r_lu, 16 * ty - p.a_lu - b_ld);
        dhi = min(15 + o_ld, 16 * ty - p.a_lu + 15 + p.b_lu);
      }
      nst[q] = dhi >= dlo ? (dhi - dlo + 4) >> 2 : 0;
      // P(x, z) = PL[(16 xt + l15) pp + z - x + lu_p],  z = x0t + dlo + 4 s + zq
      tl[q].pa = (16 * xt + l15) * pp + dlo + zq - l15 + lup;
      if (FWD) {
        // Q(z, y) = QL[(y - x0 + lu_o) qp + z - y + lu_b],  y = x0t - lu_o + 16 ty + l15
        tl[q].pb = (16 * xt + 16 * ty + l15) * qp + (dlo + r_lu - 16 * ty) + zq - l15 + p.b_lu;
      } else {
        // Q(z, y) = QL[(z - x0 + lu_o) qp + y - z + lu_b],  y = x0t - lu_a + 16 ty + l15
        tl[q].pb = (16 * xt + dlo + zq + r_lu) * qp + (16 * ty - p.a_lu - dlo) + l15 - zq + p.b_lu;
      }
    }
  }
  // result cell of accumulator element r: row 16 xt + 4 zq + r, band index 16 ty + l15 - (4 zq + r)
  const int srow = (16 * xt + 4 * zq) * Wout + l15 - 4 * zq;

  StreamRows<kSUQ, kSThreads> sq;
  StreamRows<FWD ? kSUQ : kSUP, kSThreads> sp, sr;
  const float* q_end = bt + cells_b;
  const float* p_end = pt + cells_p;
  auto make_h = [&](int x0) __attribute__((always_inline)) {
    // sp.v = g, sr.v = 1/S of the same cells: H = g / S, NaN where 1/S is marked unusable
    // (the cell was computed exactly); H goes to the workspace for grad_b as well
    float* hb = p.ws_h + (bn + x0 + sp.e0) * (long)Wp - sp.lead;
#pragma unroll
    for (int u = 0; u < (FWD ? kSUQ : kSUP); ++u) {
      const int vi = tid + kSThreads * u;
      if (vi < sp.nvec) {
        mm_f4 x = sp.v[u];
        const mm_f4 r = sr.v[u];
#pragma unroll
        for (int t = 0; t < 4; ++t) x[t] = r[t] < 0.f ? __builtin_nanf("") : x[t] * r[t];
        sp.v[u] = x;
        const int e = 4 * vi - sp.lead;
        if (e >= 0 && e + 3 < sp.count) {
          *reinterpret_cast<mm_f4*>(hb + 4 * vi) = x;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (e + t >= 0 && e + t < sp.count) hb[4 * vi + t] = x[t];
        }
      }
    }
  };
  auto load_p = [&](int x0) __attribute__((always_inline)) {
    sp.load(p_item, pt, p_end, x0, kSRows, n, Wp, tid);
    if (mk_h) sr.load(r_item, p.ws_r, p.ws_r + cells_o, x0, kSRows, n, Wp, tid);
  };
  auto store_p = [&](int x0) __attribute__((always_inline)) {
    if (mk_h) make_h(x0);
    sp.store(PL, pp, x0, kSRows, n, lup, tid);
  };

  // ---- first window: rows x0 - lu_o ... of Q in pieces of 64, the block's rows of P
  int x0 = xr0;
  for (int c = 0; c < QR; c += kSRows) {
    const int rows = min(kSRows, QR - c);
    sq.load(q_item, bt, q_end, x0 - r_lu + c, rows, n, Wb, tid);
    sq.store(QL + c * qp, qp, x0 - r_lu + c, rows, n, p.b_lu, tid);
  }
  load_p(x0);
  store_p(x0);
  if (FWD && PREP) {
    if (tid < kSRows) al[tid] = x0 + tid < n ? p.ws_al[bn + x0 + tid] : 0.f;
    for (int t = tid; t < QR; t += kSThreads) {
      const int o = x0 - r_lu + t;
      be[t] = (o >= 0 && o < n) ? p.ws_be[bn + o] : 0.f;
    }
  }
  __syncthreads();

  const float thr = fast_exp2(-kBandGuardBits);
  const unsigned omagic = (unsigned)((0x100000000ull + (unsigned)Wout - 1) / (unsigned)Wout);
  const int shift_floats = (QR - kSRows) * qp;  // the part of the window that stays

  for (; x0 < xr1; x0 += kSRows) {
    const bool more = x0 + kSRows < xr1;  // uniform
    float alv = 0.f, bev = 0.f, bemv_keep = 0.f;
    if (more) {  // the next block's new rows: reads only, they land after this block's tiles
      sq.load(q_item, bt, q_end, x0 - r_lu + QR, kSRows, n, Wb, tid);
      load_p(x0 + kSRows);
      if (FWD && PREP) {
        if (tid < kSRows && x0 + kSRows + tid < n) alv = p.ws_al[bn + x0 + kSRows + tid];
        const int o = x0 - r_lu + QR + tid - kSRows;
        if (tid >= kSRows && tid < 2 * kSRows && o >= 0 && o < n) bev = p.ws_be[bn + o];
      }
    }

    // ---- tiles
#pragma unroll
    for (int q = 0; q < kSTiles; ++q) {
      const int ty = half + 2 * q;
      if (ty < ny) {  // uniform
        mm_f4 c = mm_f4{0.f, 0.f, 0.f, 0.f};
        const float* pa = PL + tl[q].pa;
        const float* pb = QL + tl[q].pb;
        int s = nst[q];
        for (; s >= 4; s -= 4) {
          const float a0 = pa[0], a1 = pa[4], a2 = pa[8], a3 = pa[12];
          const float b0 = pb[0], b1 = pb[dq], b2 = pb[2 * dq], b3 = pb[3 * dq];
          pa += 16;
          pb += 4 * dq;
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, b0, c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, b1, c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a2, b2, c, 0, 0, 0);
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a3, b3, c, 0, 0, 0);
        }
        for (; s > 0; --s) {
          const float a0 = pa[0], b0 = pb[0];
          pa += 4;
          pb += dq;
          c = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, b0, c, 0, 0, 0);
        }
        const bool inner = 16 * ty - 15 >= 0 && 16 * ty + 15 < Wout;  // no lane of the tile is outside
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int col = 16 * ty + l15 - (4 * zq + r);
          if (inner || (col >= 0 && col < Wout)) S[srow + r * (Wout - 1) + 16 * ty] = c[r];
        }
      }
    }
    __syncthreads();  // A: the block's operands are consumed, its results are in S

    // ---- the window of the next block.  What stays of this one moves down: read, barrier,
    // write; then the new rows, which have been waiting in registers since before the tiles.
    // The block's results leave after that: their stores are then still in flight while
    // the next block's tiles run, and nothing that follows has to wait for them.
    if (more) {
      mm_f4 mv[kSShift];
#pragma unroll
      for (int u = 0; u < kSShift; ++u) {
        const int e = 4 * (tid + kSThreads * u);
        if (e < shift_floats) mv[u] = *reinterpret_cast<const mm_f4*>(QL + kSRows * qp + e);
      }
      if (FWD && PREP && tid < QR - kSRows) bemv_keep = be[tid + kSRows];
      __syncthreads();  // B: every read of the old window is done
#pragma unroll
      for (int u = 0; u < kSShift; ++u) {
        const int e = 4 * (tid + kSThreads * u);
        if (e < shift_floats) *reinterpret_cast<mm_f4*>(QL + e) = mv[u];
      }
      sq.store(QL + (QR - kSRows) * qp, qp, x0 - r_lu + QR, kSRows, n, p.b_lu, tid);
      store_p(x0 + kSRows);
    }
    // ---- rows out: one contiguous run of memory
    {
      const int rows = min(kSRows, n - x0);
      const int cells = rows * Wout;
      float* ob = p.o0 + (bn + x0) * (long)Wout;
      const float* xe = PREP && !FWD ? p.ws_ea + (bn + x0) * (long)Wout : nullptr;
      float* rb = PREP && FWD ? p.ws_r + (bn + x0) * (long)Wout : nullptr;
      const bool vec = (cells & 3) == 0 && (reinterpret_cast<uintptr_t>(ob) & 15) == 0 &&
                       (!PREP || (FWD ? (reinterpret_cast<uintptr_t>(rb) & 15) == 0
                                      : (reinterpret_cast<uintptr_t>(xe) & 15) == 0));
      const int stepc = vec ? 4 : 1;
      for (int e = stepc * tid; e < cells; e += stepc * kSThreads) {
        float sv[4], ov[4], rv[4], xv[4];
        if (vec) {
          const mm_f4 s4 = *reinterpret_cast<const mm_f4*>(S + e);
          sv[0] = s4[0]; sv[1] = s4[1]; sv[2] = s4[2]; sv[3] = s4[3];
          if (PREP && !FWD) {
            const mm_f4 x4 = *reinterpret_cast<const mm_f4*>(xe + e);
            xv[0] = x4[0]; xv[1] = x4[1]; xv[2] = x4[2]; xv[3] = x4[3];
          }
        } else {
          sv[0] = S[e];
          if (PREP && !FWD) xv[0] = xe[e];
        }
        const int r0 = (int)__umulhi((unsigned)e, omagic), k0 = e - r0 * Wout;
        unsigned redo = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          if (t < stepc) {
            const bool wrap = k0 + t >= Wout;  // Wout >= 4: one row change at most
            const int r = r0 + (wrap ? 1 : 0), k = k0 + t - (wrap ? Wout : 0);
            float v = sv[t];
            rv[t] = 0.f;
            if (FWD && PREP) {
              const int o = x0 + r + k - r_lu;
              if (o >= 0 && o < n) {
                const float sh = al[r] + be[r + k];
                if ((v >= thr) && (v < INFINITY) && (sh > 0.9f * kFloor) && (sh < INFINITY)) {
                  rv[t] = __builtin_amdgcn_rcpf(v);
                  v = __builtin_fmaf(fast_log2(v), kLn2, sh);
                } else {
                  redo |= 1u << t;
                  rv[t] = -1.f;  // tells the backward that 1/S is not usable here
                }
              } else {
                v = 0.f;  // outside the matrix: the reference's zero fill
              }
            } else {
              if (PREP) v *= xv[t];
              if (!(fabsf(v) <= FLT_MAX)) redo |= 1u << t;
            }
            ov[t] = v;
          }
        }
        if (vec) {
          *reinterpret_cast<mm_f4*>(ob + e) = mm_f4{ov[0], ov[1], ov[2], ov[3]};
          if (FWD && PREP) *reinterpret_cast<mm_f4*>(rb + e) = mm_f4{rv[0], rv[1], rv[2], rv[3]};
        } else {
          ob[e] = ov[0];
          if (FWD && PREP) rb[e] = rv[0];
        }
        if (redo) {  // rare: these cells again, from memory, by the per-cell routine (it stores them itself)
          for (int t = 0; t < stepc; ++t)
            if ((redo >> t) & 1u) {
              const bool wrap = k0 + t >= Wout;
              const int r = r0 + (wrap ? 1 : 0), k = k0 + t - (wrap ? Wout : 0);
              if (FWD) {
                if (PREP) band_fwd_cell<GENBMM_BAND_LOG>(p, bn + x0 + r, x0 + r, k);
                else band_fwd_cell<GENBMM_BAND_MUL>(p, bn + x0 + r, x0 + r, k);
              } else {
                if (PREP) band_bwd_a_cell<GENBMM_BAND_LOG>(p, bn + x0 + r, x0 + r, k);
                else band_bwd_a_cell<GENBMM_BAND_MUL>(p, bn + x0 + r, x0 + r, k);
              }
            }
        }
      }
    }
    if (!more) break;
    if (FWD && PREP) {  // maxima of the next block's rows (this block's were read by the lines above)
      __syncthreads();
      if (tid < QR - kSRows) be[tid] = bemv_keep;
      if (tid < kSRows) al[tid] = alv;
      if (tid >= kSRows && tid < 2 * kSRows) be[QR - 2 * kSRows + tid] = bev;
    }
    __syncthreads();  // C
  }
}

}  // namespace genbmm
