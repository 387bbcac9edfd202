// Banded (+,*) products on the matrix cores, operands fed from memory: forward, grad_a and
// grad_b of the plain product and of the log product on the forward's workspace.  No
// operand tiles shared through LDS, no barrier.
//
// In dense coordinates each of the three is C[i, j] = sum_k P(i, k) Q(k, j)
// cut into 16 x 16 tiles of (i, j); one wave owns a tile row (16 rows i) and walks its
// tiles along j; waves never meet.
//
//   forward  i = x, k = z, j = y   P = a[x][z - x + lu_a]    Q = b[y][z - y + lu_b]   -> out[x][y - x + lu_o]
//   grad_a   i = x, k = y, j = z   P = g[x][y - x + lu_o]    Q = b[y][z - y + lu_b]   -> ga[x][z - x + lu_a]
//   grad_b   i = y, k = x, j = z   P = g[x][y - x + lu_o]    Q = a[x][z - x + lu_a]   -> gb[y][z - y + lu_b]
//
// v_mfma_f32_16x16x4_f32 sums over four values of k; which four is free as long as both
// operands agree.  Here lane (l15, zq) feeds, in the t-th of four consecutive
// instructions, k = K + 4 zq + t, for a chunk of 16 k starting at K.  An operand is read
// in one of two ways:
//
//  * its band row is the operand's own row or column (l15) and k runs along the row (a
//    and b in the forward, g in grad_a): the four values a lane needs are four
//    neighbouring cells, and a chunk is 64 contiguous bytes of each of 16 band rows.  It
//    is read by one 16-byte load per lane (4-byte aligned) with four neighbouring
//    lanes on one row - which the memory pipeline takes as one access per row - and
//    the cells then change lanes to where the instruction wants them (ds_bpermute for
//    Q; P goes through the wave's own piece of LDS anyway).
//  * its band row is k (b in grad_a, g and a in grad_b): 16 lanes l15 read 16
//    neighbouring cells of row k - four 4-byte loads per lane for the four k, each
//    already in the lane that feeds it.
//
// k runs on a grid of chunks that starts at the first k the tile row's P can meet.  The
// wave puts its NU chunks of P into LDS once, laid out as the instruction reads them.  A
// tile uses the chunks that its cells can meet; the (tile, chunk) pairs of a tile row
// form one list, the same for every tile row of a product, which the host writes once
// and the wave walks with the loads of Q four pairs ahead of the instructions.  Every
// step of the walk issues the same memory operations whatever the pair, so that the
// waits count exactly what is in flight; the list is filled up to a multiple of four at
// its front with steps that multiply nothing.  Cells of a chunk outside a lane's band
// are multiplied by zero after the load.  Tile rows whose band cells reach outside the
// matrix, or whose loads could leave the tensors, read cell by cell from addresses held
// inside the tensor and test every cell (EDGE).
//
// The log product on the forward's workspace: the forward multiplies EA and EB and takes
// the logarithm per cell (and leaves 1/S); the gradients form H = g / S while they read g
// and multiply the sums by EA / EB on the way out.
//
// A result that is not finite (an operand that is not, against a zero of the padding; an
// H that is marked unusable), and in the forward of the log product a sum outside the
// guard, is noted per lane or per cell and recomputed from memory by the per-cell
// routine once the tile row is done.
//
// Measured at 64 x 4096 with 65 diagonals the forward issues about 1 700 instructions per
// tile row for its 100 matrix instructions and is bound by that count (a SIMD of this
// chip issues one instruction of any kind about every 4.4 cycles and nothing beside a
// matrix instruction's 32).
#pragma once

#include <cfloat>

#include "banded_flat.h"

namespace GENBMM_NS {

constexpr int kDirFwd = 0, kDirGradA = 1, kDirGradB = 2;
constexpr int kDirTiles = 32;   // tiles per tile row, at most (5 bits of a step word; a bit per cell in 128 bits)
constexpr int kDirChunks = 30;  // chunks of the first operand per tile row, at most (5 bits)
constexpr int kDirDepth = 4;    // pairs whose loads of Q are in flight
constexpr int kDirWaves = 1;    // waves (tile rows) per workgroup
constexpr int kDirMargin = 48;  // floats a load can stray from the band rows it is meant for
typedef float dir_f4u __attribute__((ext_vector_type(4), aligned(4)));

// The walk over a tile row's (tile, chunk) pairs.  One word per step:
//   bits 0-12  where the pair's cells of Q start, in units of 16 floats
//   bits 13-17 chunk of P
//   bits 18-22 tile      bit 23  the tile is complete after this step
//   bit 24  some lane's cells of Q lie past the upper end of its band (D = 0)
//   bit 25 / 26  ... below the lower end: D is the plan's lowest / the one above it
//   bit 27  a filling step (nothing to multiply)
//   bit 28  every cell of the tile is inside the result band
// (D: chunk minus tile, or tile minus chunk for an operand whose band row is k; a lane's
// cell t of Q is Wq - 1 + 16 D + s_t with s_t in [-15, 15]), and beside it the word of
// the step kDirDepth further on, whose cells of Q are asked for now.
constexpr int kDirSteps = 400;  // of a tile row (the table travels as a kernel argument: 3.2 KB)
constexpr unsigned kDirQMask = 0x1fffu;
constexpr int kDirChunkShift = 13, kDirTileShift = 18;
constexpr unsigned kDirDone = 1u << 23, kDirPastHi = 1u << 24, kDirBelowLo0 = 1u << 25, kDirBelowLo1 = 1u << 26,
                   kDirFill = 1u << 27, kDirWhole = 1u << 28;
constexpr size_t kDirLdsLimit = 160 * 1024;  // of a workgroup (one compute unit's LDS)
struct DirStep {
  unsigned now, ahead;
};
// (CAP: steps the table has room for.  Narrow bands travel in the small form - a kernel
// argument of 3 KB costs every launch a few microseconds.)
constexpr int kDirStepsSmall = 88;
template <int CAP>
struct DirPlanT {
  int steps;  // a multiple of kDirDepth
  int d_lo;   // the lowest D of the plan
  int Wp, Wq, Wout;
  int plo, phi;  // P(i, k) is inside its band for k in [i - plo, i + phi]
  int lu_out;    // out[i][j - i + lu_out]
  int NU, nt;    // chunks of P, tiles per tile row
  DirStep e[CAP + 1];
};
using DirPlan = DirPlanT<kDirSteps>;
using DirPlanSmall = DirPlanT<kDirStepsSmall>;
inline DirPlanSmall dir_plan_small(const DirPlan& g) {  // g.steps <= kDirStepsSmall
  DirPlanSmall r;
  r.steps = g.steps; r.d_lo = g.d_lo; r.Wp = g.Wp; r.Wq = g.Wq; r.Wout = g.Wout;
  r.plo = g.plo; r.phi = g.phi; r.lu_out = g.lu_out; r.NU = g.NU; r.nt = g.nt;
  for (int i = 0; i <= g.steps; ++i) r.e[i] = g.e[i];
  return r;
}

inline int dir_chunks(int Wp) { return (Wp + 30) >> 4; }  // chunks of 16 k that a tile row's P meets
// LDS of one wave: its chunks of P, 1 KB each; then the tile row's results, which leave as one
// contiguous run of memory.  The forward of the log product puts the row maxima of b for its
// tiles and of a for its rows where the chunks were, once the walk is done with them.  (LDS
// bounds the waves per compute unit, and the kernels' time follows their number: at 65
// diagonals per operand 13.4 KB per wave are twelve waves, a KB more ten.)
inline int dir_wave_lds(const DirPlan& g, int kind, bool prep) {
  return max(g.NU * 1024, kind == kDirFwd && prep ? 64 * g.nt + 64 : 0) + 64 * g.Wout;
}

inline bool dir_plan(DirPlan& g, int kind, int a_lu, int Wa, int b_lu, int Wb) {
  const int a_ld = Wa - 1 - a_lu, b_ld = Wb - 1 - b_lu;
  const int Wo = Wa + Wb - 1, r_lu = a_lu + b_ld, r_ld = Wo - 1 - r_lu;
  int qlo, qhi;  // Q(k, j) is inside its band for k in [j - qlo, j + qhi]
  if (kind == kDirFwd) {
    g.Wp = Wa; g.Wq = Wb; g.Wout = Wo; g.plo = a_lu; g.phi = a_ld; g.lu_out = r_lu; qlo = b_lu; qhi = b_ld;
  } else if (kind == kDirGradA) {
    g.Wp = Wo; g.Wq = Wb; g.Wout = Wa; g.plo = r_lu; g.phi = r_ld; g.lu_out = a_lu; qlo = b_ld; qhi = b_lu;
  } else {
    g.Wp = Wo; g.Wq = Wa; g.Wout = Wb; g.plo = r_ld; g.phi = r_lu; g.lu_out = b_lu; qlo = a_ld; qhi = a_lu;
  }
  const bool qrow = kind != kDirFwd;
  const int NU = g.NU = dir_chunks(g.Wp), nt = g.nt = (g.Wout + 30) >> 4;
  if (NU > kDirChunks || nt > kDirTiles || max(NU, nt) * g.Wq > (int)kDirQMask) return false;
  if ((size_t)kDirWaves * dir_wave_lds(g, kDirFwd, true) > kDirLdsLimit) return false;
  unsigned list[kDirTiles * kDirChunks];
  int np = 0, d_lo = 0;
  for (int pass = 0; pass < 2; ++pass) {
    np = 0;
    for (int tj = 0; tj < nt; ++tj) {
      // the tile's k relative to i0 in [dlo, dhi]; chunk u covers [16 u - plo, 16 u - plo + 15].  A
      // tile whose cells meet no k gets one chunk all the same (every product then has a zero
      // of the band masks in it).
      const int dlo = max(-g.plo, 16 * tj - g.lu_out - qlo);
      const int dhi = min(15 + g.phi, 16 * tj - g.lu_out + 15 + qhi);
      const int ulo = min(NU - 1, max(0, (dlo + g.plo) >> 4));
      const int uhi = max(ulo, min(NU - 1, (dhi + g.plo) >> 4));
      for (int u = ulo; u <= uhi; ++u) {
        const int d = qrow ? tj - u : u - tj;
        if (pass == 0) {
          d_lo = min(d_lo, d);
          continue;
        }
        // past the upper end only for D = 0, below the lower end only for the lowest two D (a
        // lane's cells of one chunk are at most 30 apart)
        const unsigned hi = d >= 0, lo = 16 * d < 16 - g.Wq;
        if (d > 0 || (lo && d > d_lo + 1)) return false;
        const unsigned whole = 16 * tj - 15 >= 0 && 16 * tj + 15 < g.Wout;
        const int q16 = qrow ? u * (g.Wq - 1) + tj : tj * (g.Wq - 1) + u;
        list[np++] = (unsigned)q16 | (unsigned)u << kDirChunkShift | (unsigned)tj << kDirTileShift |
                     (u == uhi ? kDirDone : 0u) | (hi ? kDirPastHi : 0u) | (lo && d == d_lo ? kDirBelowLo0 : 0u) |
                     (lo && d == d_lo + 1 ? kDirBelowLo1 : 0u) | (whole ? kDirWhole : 0u);
      }
    }
  }
  g.d_lo = d_lo;
  const int pad = (kDirDepth - (np & (kDirDepth - 1))) & (kDirDepth - 1);
  if (np + pad > kDirSteps) return false;
  g.steps = np + pad;
  for (int i = 0; i < pad; ++i) g.e[i].now = (list[0] & kDirQMask) | kDirFill;  // chunk 0, read and not used
  for (int i = 0; i < np; ++i) g.e[pad + i].now = list[i];
  g.e[g.steps].now = g.e[g.steps - 1].now;
  for (int i = 0; i <= g.steps; ++i) g.e[i].ahead = g.e[min(i + kDirDepth, g.steps - 1)].now;
  return true;
}

// One tile row.  All arguments but `lane` are uniform.  lds: this wave's piece.
template <int KIND, bool PREP, bool EDGE, class Plan>
__device__ __forceinline__ void dir_row(const BandArgs& p, const Plan& g, long bn, int i0, int lane, float* lds,
                                        long rows) {
  constexpr bool FWD = KIND == kDirFwd, GA = KIND == kDirGradA;
  constexpr bool PROW = KIND == kDirGradB;  // P's band row is k
  constexpr bool QROW = KIND != kDirFwd;    // Q's band row is k
  constexpr bool MKH = PREP && !FWD;        // P = g / S, formed while it is read
  constexpr bool STAGE = !EDGE;
  const int n = p.n, Wp = g.Wp, Wq = g.Wq, Wout = g.Wout, NU = g.NU, nt = g.nt;
  const int l15 = lane & 15, zq = lane >> 4;
  // a lane that loads 16 bytes: lane 4 r + c takes row r, cells 4 c .. 4 c + 3 of the chunk; the
  // instruction wants them in lane 16 c + r
  const int lr = lane >> 2, lc = lane & 3;
  const int from = 4 * (4 * l15 + zq);  // byte index of the lane this one takes its cells from
  const int K0 = i0 - g.plo;            // first k of chunk 0
  const int J0 = i0 - g.lu_out;         // first column of tile 0
  // P and Q: the workspace's factors (float) in the prepared product, else the caller's tensors
  // (element type, widened by the loads); g always is the caller's.
  // offsets from the first cell of the batch item; EDGE keeps them inside the tensor
  auto pitem = [&] {
    if constexpr (FWD && PREP) return static_cast<const float*>(p.ws_ea) + bn * (long)Wp;
    else if constexpr (FWD) return p.a + bn * (long)Wp;
    else return p.g + bn * (long)Wp;
  }();
  const float* ritem = MKH ? p.ws_r + bn * (long)Wp : nullptr;
  auto qitem = [&] {
    if constexpr (PREP) return static_cast<const float*>(KIND == kDirGradB ? p.ws_ea : p.ws_eb) + bn * (long)Wq;
    else return (KIND == kDirGradB ? p.a : p.b) + bn * (long)Wq;
  }();
  const long cells_p = rows * Wp, cells_q = rows * Wq;
  const int p_min = (int)max(-bn * (long)Wp, -(1L << 30)), p_max = (int)min(cells_p - bn * (long)Wp - 1, 1L << 30);
  const int q_min = (int)max(-bn * (long)Wq, -(1L << 30)), q_max = (int)min(cells_q - bn * (long)Wq - 1, 1L << 30);
  auto clamped = [](int v, int lo, int hi) __attribute__((always_inline)) { return min(max(v, lo), hi); };
  // H = g / S; NaN where 1/S is marked unusable (the cell's gradients are then recomputed)
  auto mk_h = [](float gv, float rv) __attribute__((always_inline)) {
    return rv < 0.f ? __builtin_nanf("") : gv * rv;
  };

  // ---- Q.  A lane's cell t is Wq - 1 + 16 D + st with
  //   band row j: loading lane (lr, lc), row J0 + 16 tj + lr, st = 4 lc - lr + t, D = u - tj
  //   band row k: lane (l15, zq), row K0 + 16 u + 4 zq + t, st = l15 - 4 zq - t, D = tj - u
  // and its cells of step (tj, u) start 16 * (bits 0-11 of the step's word) floats on.
  const int s0 = QROW ? l15 - 4 * zq : 4 * lc - lr;  // st = s0 -/+ t
  int qoff[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
    qoff[t] = QROW ? (K0 + 4 * zq + t) * (Wq - 1) + J0 + l15 + (Wq - 1 - g.plo + g.lu_out)  // k (Wq - 1) + j + lu_q
                   : (J0 + lr) * Wq + Wq - 1 + s0 + t;
  auto issue = [&](unsigned e, mm_f4& q) __attribute__((always_inline)) {
    const int soff = 16 * (int)(e & kDirQMask);  // uniform
    if (QROW || EDGE) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        int o = qoff[t] + soff;
        if (EDGE) o = clamped(o, q_min, q_max);
        q[t] = qitem[o];
      }
    } else {
      const float4 w = ld4((qitem + soff) + qoff[0]);
      q = mm_f4{w.x, w.y, w.z, w.w};
    }
  };
  // the first steps' cells of Q are asked for before anything else
  mm_f4 qraw[kDirDepth];
#pragma unroll
  for (int s = 0; s < kDirDepth; ++s) issue(g.e[s].now, qraw[s]);

  // ---- P into LDS, as the instruction reads it (lane, t).
  //   band row i: loading lane (lr, lc), row i0 + lr, cells 16 u + 4 lc - lr + t, k = K0 + 16 u + 4 lc + t
  //   band row k: lane (l15, zq), row k = K0 + 16 u + 4 zq + t, cell Wp - 1 - 16 u + l15 - 4 zq - t
  {
    mm_f4* pl = reinterpret_cast<mm_f4*>(lds);
    const int off_i = (i0 + lr) * Wp + 4 * lc - lr;                 // + 16 u + t
    const int lu_row = Wp - 1 - g.plo;  // band row k: cell = i - k + lu_row, at k (Wp - 1) + i + lu_row
    const int off_k = (K0 + 4 * zq) * (Wp - 1) + i0 + l15 + lu_row;  // + (16 u + t) (Wp - 1)
    // chunks whose loads are in flight together: all of them for bands up to 65 diagonals
    // (the registers are free: LDS, not registers, bounds the waves per compute unit)
    constexpr int kDirGroup = FWD ? 6 : 10;
    for (int u0 = 0; u0 < NU; u0 += kDirGroup) {
      mm_f4 v[kDirGroup], w[kDirGroup];
#pragma unroll
      for (int s = 0; s < kDirGroup; ++s) {
        const int u = min(u0 + s, NU - 1);  // same number of loads whatever NU
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          if (PROW || EDGE) {
            int o = PROW ? off_k + (16 * u + t) * (Wp - 1) : off_i + 16 * u + t;
            if (EDGE) o = clamped(o, p_min, p_max);
            v[s][t] = pitem[o];
            if (MKH) w[s][t] = ritem[o];
          }
        }
        if (!PROW && !EDGE) {
          const float4 x = ld4(pitem + (off_i + 16 * u));
          v[s] = mm_f4{x.x, x.y, x.z, x.w};
          if (MKH) {
            const dir_f4u y = *reinterpret_cast<const dir_f4u*>(ritem + (off_i + 16 * u));
            w[s] = mm_f4{y[0], y[1], y[2], y[3]};
          }
        }
      }
#pragma unroll
      for (int s = 0; s < kDirGroup; ++s) {
        const int u = u0 + s;
        if (u < NU) {
          mm_f4 x = v[s];
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int cell = PROW ? Wp - 1 - 16 * u + l15 - 4 * zq - t : 16 * u + 4 * lc - lr + t;
            bool ok = (unsigned)cell < (unsigned)Wp;
            if (EDGE) {
              const int k = K0 + 16 * u + (PROW ? 4 * zq : 4 * lc) + t;
              ok = ok && i0 + (PROW ? l15 : lr) < n && (unsigned)k < (unsigned)n;
            }
            const float val = MKH ? mk_h(x[t], w[s][t]) : x[t];
            x[t] = ok ? val : 0.f;
          }
          pl[64 * u + (PROW ? lane : 16 * lc + lr)] = x;
        }
      }
    }
  }
  // the tile row's 16 x Wout results, in the last 64 Wout bytes of the wave's piece
  float* aux = lds + ((FWD && PREP) ? max(256 * NU, 16 * nt + 16) : 256 * NU);
  // forward of the log product: beta of every column the wave's tiles cover and alpha of its 16
  // rows, asked for now, put into LDS over the chunks when the walk is over
  float* bet = lds;
  float* alp = lds + 16 * nt;
  float betr[kDirTiles / 4], alpr = 0.f;
  if (FWD && PREP) {
#pragma unroll
    for (int s = 0; s < kDirTiles / 4; ++s) {
      const int t = lane + 64 * s, y = J0 + t;
      betr[s] = t < 16 * nt && (unsigned)y < (unsigned)n ? p.ws_be[bn + y] : 0.f;
    }
    if (lane < 16) alpr = i0 + lane < n ? p.ws_al[bn + i0 + lane] : 0.f;
  }

  // Factors 1 / 0 for the cells of a chunk at the ends of Q's band: past the upper end
  // (cell >= Wq) only for D = 0; below the lower end (cell < 0) for the lowest one or two D.
  float m_hi[4], m_lo0[4], m_lo1[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int st = QROW ? s0 - t : s0 + t;
    m_hi[t] = st <= 0 ? 1.f : 0.f;
    m_lo0[t] = Wq - 1 + 16 * g.d_lo + st >= 0 ? 1.f : 0.f;
    m_lo1[t] = Wq - 1 + 16 * (g.d_lo + 1) + st >= 0 ? 1.f : 0.f;
  }
  // the loaded cells of step e, zero where the lane is outside the band (EDGE: or the matrix).
  // (A factor 0 on a cell that is not finite leaves a NaN, which the test of the result catches;
  // the cell belongs to a neighbouring band row.)
  auto mask = [&](unsigned e, mm_f4& x) __attribute__((always_inline)) {
    if (EDGE) {
      const int tj = (e >> kDirTileShift) & 31u, u = (e >> kDirChunkShift) & 31u;
      const int D = QROW ? tj - u : u - tj;
      const int j = J0 + 16 * tj + (QROW ? l15 : lr);
      const int k = K0 + 16 * u + (QROW ? 4 * zq : 4 * lc);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int cell = Wq - 1 + 16 * D + (QROW ? s0 - t : s0 + t);
        const bool ok = (unsigned)cell < (unsigned)Wq && (unsigned)j < (unsigned)n && (unsigned)(k + t) < (unsigned)n;
        x[t] = ok ? x[t] : 0.f;
      }
    } else {
      if (e & kDirPastHi) {  // uniform
        asm volatile("" ::: "memory");  // keeps this a branch: most steps have nothing to mask
#pragma unroll
        for (int t = 0; t < 4; ++t) x[t] *= m_hi[t];
      }
      if (e & kDirBelowLo0) {  // uniform
        asm volatile("" ::: "memory");
#pragma unroll
        for (int t = 0; t < 4; ++t) x[t] *= m_lo0[t];
      }
      if (e & kDirBelowLo1) {  // uniform
        asm volatile("" ::: "memory");
#pragma unroll
        for (int t = 0; t < 4; ++t) x[t] *= m_lo1[t];
      }
    }
  };
  auto to_mfma = [&](const mm_f4& v) __attribute__((always_inline)) {
    if (QROW) return v;
    const float r0 = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(v[0])));
    const float r1 = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(v[1])));
    const float r2 = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(v[2])));
    const float r3 = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(v[3])));
    return mm_f4{r0, r1, r2, r3};
  };
  const mm_f4* pl = reinterpret_cast<const mm_f4*>(lds) + lane;

  // ---- results: accumulator element r is row i0 + 4 zq + r, column J0 + 16 tj + l15,
  // band cell jj = 16 tj + l15 - 4 zq - r
  const float thr = fast_exp2(-kBandGuardBits);
  elem_t* dst = KIND == kDirGradB ? p.o1 : p.o0;
  elem_t* orow = dst + (bn + i0) * (long)Wout;
  float* rrow = FWD && PREP ? p.ws_r + (bn + i0) * (long)Wout : nullptr;
  const float* erow = MKH ? (GA ? p.ws_ea : p.ws_eb) + (bn + i0) * (long)Wout : nullptr;  // factor on the way out
  unsigned ooff[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) ooff[r] = (unsigned)((4 * zq + r) * (Wout - 1) + l15);
  float al[4] = {0.f, 0.f, 0.f, 0.f};
  if (FWD && PREP) {
#pragma unroll
    for (int r = 0; r < 4; ++r) al[r] = i0 + 4 * zq + r < n ? p.ws_al[bn + i0 + 4 * zq + r] : 0.f;
  }
  // the factors that the staged results of the log product's gradients leave with: asked for
  // now, used when the tile row is done (16 bytes per lane and round of the final copy)
  constexpr int kDirEf = 6;
  mm_f4 ef[kDirEf];
  if (MKH && STAGE) {
#pragma unroll
    for (int s = 0; s < kDirEf; ++s) {
      const dir_f4u f = *reinterpret_cast<const dir_f4u*>(erow + 4 * min(lane + 64 * s, 4 * Wout - 1));
      ef[s] = mm_f4{f[0], f[1], f[2], f[3]};
    }
  }
  const bool tail = i0 + 15 > n - 1;                   // rows beyond the matrix in this tile row
  const bool y_all = J0 >= 0 && J0 + 16 * nt - 1 < n;  // every column of every tile inside the matrix
  // cells to recompute: the forward of the log product keeps a bit per cell (bit 4 tj + r), the
  // others one flag per lane (all the lane's cells are then done again)
  unsigned __int128 redo = 0;
  float worst = 0.f;  // stays 0 while every sum is finite
  // Tile rows away from the edges collect their 16 x Wout results in LDS (aux) and write
  // them as one contiguous run of memory; the forward of the log product collects its sums S
  // there and forms out and 1/S while it copies them out (staging both values, twice the
  // LDS, measured 10 % slower than no staging at all).
  const bool plain_rows = STAGE && y_all;
  auto finish = [&](unsigned e, const mm_f4& c) __attribute__((always_inline)) {
    const int tj = (e >> kDirTileShift) & 31u;
    if (plain_rows) {  // uniform: nothing to test but the values
      const float s = (c[0] + c[1]) + (c[2] + c[3]);  // not finite if a cell is not (or the sum overflows: no harm)
      worst = __builtin_fmaf(s, 0.f, worst);          // 0 * s is NaN exactly when s is not finite
      float* st = aux + 16 * tj;
      if (e & kDirWhole) {
#pragma unroll
        for (int r = 0; r < 4; ++r) st[ooff[r]] = c[r];
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int jj = 16 * tj + l15 - 4 * zq - r;
          if (jj >= 0 && jj < Wout) st[ooff[r]] = c[r];
        }
      }
      return;
    }
    const bool whole = (e & kDirWhole) && !tail;
    const int y = J0 + 16 * tj + l15;
    const bool y_in = y_all || (unsigned)y < (unsigned)n;
    unsigned bits = 0;
    float be = 0.f;
    if (FWD && PREP) be = y_in ? p.ws_be[bn + y] : 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int jj = 16 * tj + l15 - 4 * zq - r;
      if (whole || (i0 + 4 * zq + r < n && jj >= 0 && jj < Wout)) {
        float v = y_in ? c[r] : 0.f;  // outside the matrix: the reference's zero fill
        if (FWD && PREP) {
          float rv = 0.f;
          if (y_in) {
            const float sh = al[r] + be;
            const bool ok = (v >= thr) && (v < INFINITY) && (sh >= kFloor) && (sh < INFINITY);
            rv = ok ? __builtin_amdgcn_rcpf(v) : -1.f;  // -1 tells the backward that 1/S is not usable here
            v = __builtin_fmaf(fast_log2(v), kLn2, sh);
            if (!ok) bits |= 1u << r;
          }
          (rrow + 16 * tj)[ooff[r]] = rv;
        } else {
          if (!(fabsf(v) <= FLT_MAX)) redo = 1;
          if (MKH && !STAGE) v *= (erow + 16 * tj)[ooff[r]];
        }
        if (STAGE) (aux + 16 * tj)[ooff[r]] = v;
        else (orow + 16 * tj)[ooff[r]] = to_elem<elem_t>(v);
      }
    }
    if (FWD && PREP) redo |= (unsigned __int128)bits << (4 * tj);
  };

  // ---- the walk: the loads of Q run kDirDepth steps ahead (past the end they repeat the
  // last step's and are never used); the words of the plan are read a step before their use
  const int steps = g.steps;
  mm_f4 c = mm_f4{0.f, 0.f, 0.f, 0.f};
  DirStep w = g.e[0];
  for (int i = 0; i < steps; i += kDirDepth) {
#pragma unroll
    for (int s = 0; s < kDirDepth; ++s) {
      const DirStep cur = w;
      w = g.e[i + s + 1];  // one entry past the last exists
      const unsigned e = cur.now;
      mask(e, qraw[s]);
      const mm_f4 qv = to_mfma(qraw[s]);
      const mm_f4 pv = pl[64 * ((e >> kDirChunkShift) & 31u)];
      issue(cur.ahead, qraw[s]);
      if (!(e & kDirFill)) {  // uniform: not one of the filling steps
#pragma unroll
        for (int t = 0; t < 4; ++t) c = __builtin_amdgcn_mfma_f32_16x16x4f32(pv[t], qv[t], c, 0, 0, 0);
      }
      if (e & kDirDone) {  // uniform: the tile is complete
        finish(e, c);
        c = mm_f4{0.f, 0.f, 0.f, 0.f};
      }
    }
  }

  if (FWD && PREP && plain_rows) {
#pragma unroll
    for (int s = 0; s < kDirTiles / 4; ++s)
      if (lane + 64 * s < 16 * nt) bet[lane + 64 * s] = betr[s];
    if (lane < 16) alp[lane] = alpr;
    // The sums S of the tile row are in LDS: out = log S + alpha + beta and 1/S leave as two
    // contiguous runs, four cells per lane.  A cell outside the guard gets 1/S = -1 (not usable,
    // the backward then takes the exact way) and its value from the per-cell routine right
    // behind the store (same lane, same address: in order).
    const mm_f4* so4 = reinterpret_cast<const mm_f4*>(aux);
    const float rw = 1.f / (float)Wout;
    for (int i = lane; i < 4 * Wout; i += 64) {
      const mm_f4 sv = so4[i];
      int row = (int)((float)(4 * i) * rw);  // 4 i / Wout, exact after one correction either way
      int jj = 4 * i - row * Wout;
      if (jj < 0) { --row; jj += Wout; }
      if (jj >= Wout) { ++row; jj -= Wout; }
      mm_f4 ov, rv;
      unsigned bad = 0;
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        const float sh = alp[row] + bet[row + jj], v = sv[c4];
        const bool ok = (v >= thr) && (v < INFINITY) && (sh >= kFloor) && (sh < INFINITY);
        rv[c4] = ok ? __builtin_amdgcn_rcpf(v) : -1.f;
        ov[c4] = __builtin_fmaf(fast_log2(v), kLn2, sh);
        if (!ok) bad |= 0x80000000u >> c4;
        if (++jj == Wout) { jj = 0; ++row; }
      }
      st4(orow + 4 * i, make_float4(ov[0], ov[1], ov[2], ov[3]));
      *reinterpret_cast<dir_f4u*>(rrow + 4 * i) = dir_f4u{rv[0], rv[1], rv[2], rv[3]};
      if (bad) {  // rare
        int r2 = (int)((float)(4 * i) * rw), j2 = 4 * i - r2 * Wout;
        if (j2 < 0) { --r2; j2 += Wout; }
        if (j2 >= Wout) { ++r2; j2 -= Wout; }
        for (int c4 = 0; c4 < 4; ++c4) {
          if (bad & (0x80000000u >> c4)) band_fwd_cell<GENBMM_BAND_LOG>(p, bn + i0 + r2, i0 + r2, j2);
          if (++j2 == Wout) { j2 = 0; ++r2; }
        }
      }
    }
  } else if (STAGE) {  // the tile row's 16 Wout results: one contiguous run of memory
    const mm_f4* so4 = reinterpret_cast<const mm_f4*>(aux);
#pragma unroll
    for (int s = 0; s < kDirEf; ++s) {
      const int i = lane + 64 * s;
      if (i < 4 * Wout) {
        mm_f4 v = so4[i];
        if (MKH) v = mm_f4{v[0] * ef[s][0], v[1] * ef[s][1], v[2] * ef[s][2], v[3] * ef[s][3]};
        st4(orow + 4 * i, make_float4(v[0], v[1], v[2], v[3]));
      }
    }
    for (int i = lane + 64 * kDirEf; i < 4 * Wout; i += 64) {
      mm_f4 v = so4[i];
      if (MKH) {
        const dir_f4u f = *reinterpret_cast<const dir_f4u*>(erow + 4 * i);
        v = mm_f4{v[0] * f[0], v[1] * f[1], v[2] * f[2], v[3] * f[3]};
      }
      st4(orow + 4 * i, make_float4(v[0], v[1], v[2], v[3]));
    }
  }

  // ---- cells to recompute (rare).  The stores above are to the same addresses from the
  // same lane: they stay in order.
  if (!(FWD && PREP) && !(worst == 0.f)) redo = 1;
  if (__builtin_amdgcn_ballot_w64(redo != 0) != 0) {
    if (STAGE) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // the run above was written by other lanes
    if (!(FWD && PREP) && redo) redo = ~(unsigned __int128)0;
    while (redo) {
      const unsigned long long half = (unsigned long long)redo;
      const int bit = half ? __builtin_ctzll(half) : 64 + __builtin_ctzll((unsigned long long)(redo >> 64));
      redo &= redo - 1;
      const int tj = bit >> 2, r = bit & 3;
      const int i = i0 + 4 * zq + r, jj = 16 * tj + l15 - 4 * zq - r;
      if (tj < nt && i < n && jj >= 0 && jj < Wout) {
        if (FWD) {
          if (PREP) band_fwd_cell<GENBMM_BAND_LOG>(p, bn + i, i, jj);
          else band_fwd_cell<GENBMM_BAND_MUL>(p, bn + i, i, jj);
        } else if (GA) {
          if (PREP) band_bwd_a_cell<GENBMM_BAND_LOG>(p, bn + i, i, jj);
          else band_bwd_a_cell<GENBMM_BAND_MUL>(p, bn + i, i, jj);
        } else {
          if (PREP) band_bwd_b_cell<GENBMM_BAND_LOG>(p, bn + i, i, jj);
          else band_bwd_b_cell<GENBMM_BAND_MUL>(p, bn + i, i, jj);
        }
      }
    }
  }
}

// One wave per tile row, kDirWaves tile rows per workgroup: the tile rows of workgroup `blk` of a
// product.  blocks: workgroups per batch item; wave_lds: bytes of LDS per wave; rows: band rows of
// every tensor (batch * n).
template <int KIND, bool PREP, class Plan>
__device__ __forceinline__ void dir_block(const BandArgs& p, const Plan& g, int blk, int blocks, long rows,
                                          int wave_lds, float* dir_smem) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int batch = blk / blocks;
  const int i0 = ((blk - batch * blocks) * kDirWaves + wave) * 16;
  const int n = p.n;
  if (i0 >= n) return;
  const long bn = (long)batch * n;
  float* lds = dir_smem + wave * (wave_lds >> 2);
  // May the wave take its loads as they come and skip the tests against the matrix?  Every band
  // cell of its rows of P inside the matrix (a cell of Q that is not then only ever meets a
  // zero), and the cells that the loads can touch beside the band rows inside the tensors.
  constexpr bool PROW = KIND == kDirGradB, QROW = KIND != kDirFwd;
  const long K0 = bn + i0 - g.plo, J0 = bn + i0 - g.lu_out;
  const long rp0 = PROW ? K0 : bn + i0, rp1 = PROW ? K0 + 16 * g.NU : bn + i0 + 16;  // band rows of P, of Q
  const long rq0 = QROW ? K0 : J0, rq1 = QROW ? K0 + 16 * g.NU : J0 + 16 * g.nt;
  const bool inside_matrix = i0 - g.plo >= 0 && i0 + 15 + g.phi <= n - 1;
  const bool inside_tensor = rp0 * g.Wp >= kDirMargin && rp1 * g.Wp + kDirMargin <= rows * g.Wp &&
                             rq0 * g.Wq >= kDirMargin && rq1 * g.Wq + kDirMargin <= rows * g.Wq;
  if (inside_matrix && inside_tensor) dir_row<KIND, PREP, false>(p, g, bn, i0, lane, lds, rows);
  else dir_row<KIND, PREP, true>(p, g, bn, i0, lane, lds, rows);
}

template <int KIND, bool PREP, class Plan>
__global__ __launch_bounds__(64 * kDirWaves) void k_band_dir(const BandArgs p, const Plan g, int blocks, int nblocks,
                                                            long rows, int wave_lds) {
  extern __shared__ __attribute__((aligned(16))) float dir_smem[];
  dir_block<KIND, PREP>(p, g, xcd_renumber(blockIdx.x, nblocks), blocks, rows, wave_lds, dir_smem);
}

// Both gradients in one launch, workgroup by workgroup in turn: grad_a and grad_b of
// neighbouring rows read the same rows of g (and of 1 / S), which then come from memory once.
// nblocks: workgroups of one gradient.
template <bool PREP, class Plan>
__global__ __launch_bounds__(64 * kDirWaves) void k_band_dir_grads(const BandArgs p, const Plan ga, const Plan gb,
                                                                  int blocks, int nblocks, long rows, int wave_lds) {
  extern __shared__ __attribute__((aligned(16))) float dir_smem[];
  const int v = xcd_renumber(blockIdx.x, 2 * nblocks);
  if ((v & 1) == 0) dir_block<kDirGradA, PREP>(p, ga, v >> 1, blocks, rows, wave_lds, dir_smem);
  else dir_block<kDirGradB, PREP>(p, gb, v >> 1, blocks, rows, wave_lds, dir_smem);
}

}  // namespace GENBMM_NS
