// Banded (+,*) forward on the matrix cores, operands fed from memory: no operand tiles
// shared through LDS, no barrier.
//
// Dense coordinates as in banded_mfma.h: C[x, y] = sum_z P(x, z) Q(z, y) with
// P(x, z) = a[x][z - x + lu_a] and Q(z, y) = b[y][z - y + lu_b], 16 x 16 tiles of (x, y).
// One wave owns a tile row (16 rows x) and walks its tiles along y; waves never meet.
//
// v_mfma_f32_16x16x4_f32 sums over four values of z; which four is free as long as both
// operands agree.  Here lane (l15, zq) feeds, in the t-th of four consecutive
// instructions, z = Z + 4 zq + t: the four values a lane needs for the four
// instructions are four neighbouring cells of its band row, for P (lane l15 is row x)
// and for Q (lane l15 is row y of b) alike.  A chunk of 16 z is thus 64 contiguous
// bytes of each of 16 band rows: it is read by one 16-byte load per lane (4-byte
// aligned) with four neighbouring lanes on one row - which the memory pipeline takes as
// one access per row - and the cells then change lanes to where the instruction wants
// them: P once per tile row through the wave's own piece of LDS, Q by ds_bpermute.
//
// z runs on a grid of such chunks that starts at x0 - lu_a for the tile row at x0.  A
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
// A result that is not finite (an operand that is not, against a zero of the padding),
// and in the prepared log product a sum outside the guard, is noted per lane or per cell
// and recomputed from memory by the per-cell routine once the tile row is done.
//
// Measured at 64 x 4096 with 65 diagonals the kernel issues about 1 700 instructions per
// tile row for its 100 matrix instructions and is bound by that count (a SIMD of this
// chip issues one instruction of any kind about every 4.4 cycles and nothing beside a
// matrix instruction's 32).
#pragma once

#include <cfloat>

#include "banded_mfma.h"

namespace genbmm {

constexpr int kDirTiles = 16;   // tiles per tile row, at most (a bit per cell in 64 bits)
constexpr int kDirChunks = 6;   // chunks of the first operand per tile row, at most
constexpr int kDirDepth = 4;    // pairs whose loads are in flight
typedef float dir_f4u __attribute__((ext_vector_type(4), aligned(4)));

constexpr int kDirWaves = 2;    // waves (tile rows) per workgroup

inline int dir_chunks(int Wp) { return (Wp + 30) >> 4; }  // chunks of 16 z that a tile row's P meets
// LDS of one wave: its chunks of P and one of zeros, 1 KB each; then the row maxima of b for
// its tiles (prepared log product) or the tile row's results (plain product), which then
// leave as one contiguous run of memory
inline int dir_wave_lds(int Wa, int Wo, bool prep) {
  return (dir_chunks(Wa) + 1) * 1024 + (prep ? 64 * ((Wo + 30) >> 4) : 64 * Wo);
}

// The walk over a tile row's (tile, chunk) pairs is the same for every tile row of a
// product: the host lists it once.  One word per step:
//   bits 0-11  (ty (Wb - 1) + u): where the pair's cells of Q start, in units of 16 floats
//   bits 12-14 chunk of P (the one past the last holds zeros)
//   bits 15-18 tile ty          bit 19  the tile is complete after this step
//   bit 20 / 21  some lane's cells lie past the upper / lower end of the band of b
//   bits 22-26 (u - ty) + 16    bit 27  a filling step (nothing to multiply)
//   (bit 21: u - ty is the plan's lowest, bit 28: the one above it)
//   bit 29  every cell of the tile is inside the result band
// and beside it the word of the step kDirDepth further on, whose cells of Q are asked for now.
constexpr int kDirSteps = 64;
struct DirStep {
  unsigned now, ahead;
};
struct DirPlan {
  int steps;  // a multiple of kDirDepth
  int d_lo;   // the lowest u - ty of the plan
  DirStep e[kDirSteps + 1];
};

inline bool dir_plan(DirPlan& plan, int a_lu, int Wa, int b_lu, int Wb, int r_lu, int Wo) {
  const int NU = dir_chunks(Wa), ny = (Wo + 30) >> 4;
  const int a_ld = Wa - 1 - a_lu, b_ld = Wb - 1 - b_lu;
  if (NU > kDirChunks || ny > kDirTiles || 15 * (Wb - 1) + NU >= 4096) return false;
  unsigned list[kDirTiles * kDirChunks];
  int np = 0, d_lo = 0;
  for (int ty = 0; ty < ny; ++ty) {
    const int dlo = max(-a_lu, 16 * ty - r_lu - b_lu);
    const int ulo = min(NU - 1, (dlo + a_lu) >> 4);
    d_lo = min(d_lo, ulo - ty);
  }
  plan.d_lo = d_lo;
  for (int ty = 0; ty < ny; ++ty) {
    // the tile's z relative to x0 in [dlo, dhi]; chunk u covers [16 u - lu_a, 16 u - lu_a + 15].  A
    // tile whose cells meet no z gets one chunk all the same (every product then has a zero
    // of the band masks in it).
    const int dlo = max(-a_lu, 16 * ty - r_lu - b_lu);
    const int dhi = min(15 + a_ld, 16 * ty - r_lu + 15 + b_ld);
    const int ulo = min(NU - 1, (dlo + a_lu) >> 4);
    const int uhi = max(ulo, min(NU - 1, (dhi + a_lu) >> 4));
    for (int u = ulo; u <= uhi; ++u) {
      const int d = u - ty;
      if (d + 16 < 0 || d + 16 > 31) return false;
      // below the lower end: only the plan's lowest two u - ty can be (30 cells apart at most)
      const unsigned hi = d >= 0, lo = 16 * d < 16 - Wb;
      if (d > 0 || (lo && d > d_lo + 1)) return false;
      const unsigned whole = 16 * ty - 15 >= 0 && 16 * ty + 15 < Wo;
      list[np++] = (unsigned)(ty * (Wb - 1) + u) | (unsigned)u << 12 | (unsigned)ty << 15 |
                   (unsigned)(u == uhi) << 19 | hi << 20 | (unsigned)(lo && d == d_lo) << 21 |
                   (unsigned)(d + 16) << 22 | (unsigned)(lo && d == d_lo + 1) << 28 | whole << 29;
    }
  }
  const int pad = (kDirDepth - (np & (kDirDepth - 1))) & (kDirDepth - 1);
  if (np + pad > kDirSteps) return false;
  plan.steps = np + pad;
  for (int i = 0; i < pad; ++i)
    plan.e[i].now = (list[0] & 0xfffu) | (unsigned)NU << 12 | (list[0] & (31u << 22)) | 1u << 27;
  for (int i = 0; i < np; ++i) plan.e[pad + i].now = list[i];
  plan.e[plan.steps].now = plan.e[plan.steps - 1].now;
  for (int i = 0; i <= plan.steps; ++i) plan.e[i].ahead = plan.e[min(i + kDirDepth, plan.steps - 1)].now;
  return true;
}

// One tile row.  All arguments but `lane` are uniform.  lds: this wave's piece.
template <bool PREP, bool EDGE>
__device__ __forceinline__ void dir_fwd_row(const BandArgs& p, const DirPlan& plan, long bn, int x0, int lane,
                                            float* lds, long cells_a, long cells_b) {
  const int n = p.n, Wa = p.Wa, Wb = p.Wb, Wo = p.Wo, r_lu = p.r_lu, a_lu = p.a_lu;
  const int NU = (Wa + 30) >> 4, ny = (Wo + 30) >> 4;
  const int l15 = lane & 15, zq = lane >> 4;
  // loading lane 4 r + c: row r, cells 4 c .. 4 c + 3 of the chunk; the instruction wants
  // them in lane 16 c + r
  const int lr = lane >> 2, lc = lane & 3;
  const int from = 4 * (4 * l15 + zq);  // byte index of the lane this one takes its cells from
  const int y0 = x0 - r_lu;             // first column of tile 0
  const float* at = PREP ? p.ws_ea : p.a;
  const float* bt = PREP ? p.ws_eb : p.b;
  // offsets from the first cell of the batch item; EDGE keeps them inside the tensor
  const float* aitem = at + bn * (long)Wa;
  const float* bitem = bt + bn * (long)Wb;
  const int a_min = (int)max(-bn * (long)Wa, -(1L << 30)), a_max = (int)min(cells_a - bn * (long)Wa - 1, 1L << 30);
  const int b_min = (int)max(-bn * (long)Wb, -(1L << 30)), b_max = (int)min(cells_b - bn * (long)Wb - 1, 1L << 30);
  auto clamped = [](int v, int lo, int hi) __attribute__((always_inline)) { return min(max(v, lo), hi); };

  // ---- P: row x0 + lr, cells k = 16 u + 4 lc - lr + t at dense position x0 - lu_a + 16 u + 4 lc + t,
  // to LDS where lane 16 lc + lr will read them as 16 bytes; after the last chunk one of zeros
  {
    const int kb = 4 * lc - lr;
    const int off = (x0 + lr) * Wa + kb;
    mm_f4 v[kDirChunks];
#pragma unroll
    for (int u = 0; u < kDirChunks; ++u) {
      const int uu = min(u, NU - 1);  // same number of loads whatever NU
      if (EDGE) {
#pragma unroll
        for (int t = 0; t < 4; ++t) v[u][t] = aitem[clamped(off + 16 * uu + t, a_min, a_max)];
      } else {
        const dir_f4u w = *reinterpret_cast<const dir_f4u*>(aitem + (off + 16 * uu));
        v[u] = mm_f4{w[0], w[1], w[2], w[3]};
      }
    }
    mm_f4* pl = reinterpret_cast<mm_f4*>(lds) + (16 * lc + lr);
#pragma unroll
    for (int u = 0; u < kDirChunks; ++u) {
      if (u < NU) {
        mm_f4 x = v[u];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          bool ok = (unsigned)(kb + 16 * u + t) < (unsigned)Wa;
          if (EDGE) ok = ok && x0 + lr < n && (unsigned)(x0 - a_lu + 16 * u + 4 * lc + t) < (unsigned)n;
          x[t] = ok ? x[t] : 0.f;
        }
        pl[64 * u] = x;
      }
    }
    reinterpret_cast<mm_f4*>(lds)[64 * NU + lane] = mm_f4{0.f, 0.f, 0.f, 0.f};
  }
  // behind the chunks: beta of every column the wave's tiles cover (prepared log product), or
  // the tile row's 16 x Wo results (plain product)
  float* aux = lds + 256 * (NU + 1);
  if (PREP) {
    for (int t = lane; t < 16 * ny; t += 64) {
      const int y = y0 + t;
      aux[t] = (unsigned)y < (unsigned)n ? p.ws_be[bn + y] : 0.f;
    }
  }

  // ---- Q(z, y) = b[y][k2], k2 = z - y + lu_b = 16 (u - ty) + 4 lc - lr + t + (Wb - 1) in the
  // loading lane, which takes row y = y0 + 16 ty + lr
  const int kq = 4 * lc - lr + Wb - 1;
  const int qoff = (y0 + lr) * Wb + kq;  // pair (0, 0), t = 0
  constexpr int kBias = 64;              // kq >= -15 + Wb - 1: offsets from (row y0's first cell - kBias) are unsigned
  const float* qbase = bitem + (long)y0 * Wb - kBias;
  const unsigned qlane = (unsigned)(lr * Wb + kq + kBias);
  auto issue = [&](unsigned soff16, mm_f4& q) __attribute__((always_inline)) {
    const unsigned soff = 16u * (soff16 & 0xfffu);  // uniform
    if (EDGE) {
#pragma unroll
      for (int t = 0; t < 4; ++t) q[t] = bitem[clamped(qoff + (int)soff + t, b_min, b_max)];
    } else {
      const dir_f4u w = *reinterpret_cast<const dir_f4u*>((qbase + soff) + qlane);
      q = mm_f4{w[0], w[1], w[2], w[3]};
    }
  };
  // Factors 1 / 0 for the cells of a chunk at the ends of the band of b: a lane's cell t of a
  // chunk with u - ty = d is b[y][k2], k2 = kq + 16 d + t.  Past the upper end (k2 >= Wb) only
  // for d = 0; below the lower end (k2 < 0) for the lowest one or two d of the plan.
  float m_hi[4], m_lo0[4], m_lo1[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    m_hi[t] = kq + t < Wb ? 1.f : 0.f;
    m_lo0[t] = kq + 16 * plan.d_lo + t >= 0 ? 1.f : 0.f;
    m_lo1[t] = kq + 16 * (plan.d_lo + 1) + t >= 0 ? 1.f : 0.f;
  }
  // the loaded cells of step e, zero where the lane is outside the band (EDGE: or the matrix).
  // (A factor 0 on a cell that is not finite leaves a NaN, which the test of the result catches;
  // the cell belongs to a neighbouring band row.)
  auto mask = [&](unsigned e, mm_f4& x) __attribute__((always_inline)) {
    if (EDGE) {
      const int k2 = kq + 16 * ((int)((e >> 22) & 31u) - 16);
      const int ty = (e >> 15) & 15u, u = (e >> 12) & 7u;
      const int y = y0 + 16 * ty + lr, z = x0 - a_lu + 16 * u + 4 * lc;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const bool ok = (unsigned)(k2 + t) < (unsigned)Wb && (unsigned)y < (unsigned)n && (unsigned)(z + t) < (unsigned)n;
        x[t] = ok ? x[t] : 0.f;
      }
    } else {
      if (e & (1u << 20)) {  // uniform
        asm volatile("" ::: "memory");  // keeps this a branch: most steps have nothing to mask
#pragma unroll
        for (int t = 0; t < 4; ++t) x[t] *= m_hi[t];
      }
      if (e & (1u << 21)) {  // uniform
        asm volatile("" ::: "memory");  // keeps this a branch: most steps have nothing to mask
#pragma unroll
        for (int t = 0; t < 4; ++t) x[t] *= m_lo0[t];
      }
      if (e & (1u << 28)) {  // uniform
        asm volatile("" ::: "memory");  // keeps this a branch: most steps have nothing to mask
#pragma unroll
        for (int t = 0; t < 4; ++t) x[t] *= m_lo1[t];
      }
    }
  };
  auto to_mfma = [&](const mm_f4& v) __attribute__((always_inline)) {
    const float r0 = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(v[0])));
    const float r1 = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(v[1])));
    const float r2 = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(v[2])));
    const float r3 = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(v[3])));
    return mm_f4{r0, r1, r2, r3};
  };
  const mm_f4* pl = reinterpret_cast<const mm_f4*>(lds) + lane;

  // ---- results: accumulator element r is row x0 + 4 zq + r, column y0 + 16 ty + l15,
  // band cell j = 16 ty + l15 - 4 zq - r
  const float thr = fast_exp2(-kBandGuardBits);
  float* orow = p.o0 + (bn + x0) * (long)Wo;
  float* rrow = PREP ? p.ws_r + (bn + x0) * (long)Wo : nullptr;
  unsigned ooff[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) ooff[r] = (unsigned)((4 * zq + r) * (Wo - 1) + l15);
  float al[4] = {0.f, 0.f, 0.f, 0.f};
  if (PREP) {
#pragma unroll
    for (int r = 0; r < 4; ++r) al[r] = x0 + 4 * zq + r < n ? p.ws_al[bn + x0 + 4 * zq + r] : 0.f;
  }
  const bool tail = x0 + 15 > n - 1;                   // rows beyond the matrix in this tile row
  const bool y_all = y0 >= 0 && y0 + 16 * ny - 1 < n;  // every column of every tile inside the matrix
  // cells to recompute: the prepared log product keeps a bit per cell (bit 4 ty + r), the plain
  // product one flag per lane (all the lane's cells are then done again)
  unsigned long long redo = 0;
  float worst = 0.f;  // plain product: stays 0 while every result is finite
  // The plain product's tile rows away from the edges collect their 16 x Wo results in LDS
  // (aux) and write them as one contiguous run of memory.  (Measured for the prepared log
  // product too, with 1/S beside: the LDS it takes leaves three waves per compute unit fewer
  // and the kernel 10 % slower.)
  constexpr bool STAGE = !PREP && !EDGE;
  float* st_o = aux;
  const bool plain_rows = !PREP && !EDGE && y_all;
  auto finish = [&](unsigned e, const mm_f4& c) __attribute__((always_inline)) {
    const int ty = (e >> 15) & 15u;
    if (plain_rows) {  // uniform: nothing to test but the values
      const float s = (c[0] + c[1]) + (c[2] + c[3]);  // not finite if a cell is not (or the sum overflows: no harm)
      worst = __builtin_fmaf(s, 0.f, worst);          // 0 * s is NaN exactly when s is not finite
      float* st = st_o + 16 * ty;
      if (e & (1u << 29)) {
#pragma unroll
        for (int r = 0; r < 4; ++r) st[ooff[r]] = c[r];
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int j = 16 * ty + l15 - 4 * zq - r;
          if (j >= 0 && j < Wo) st[ooff[r]] = c[r];
        }
      }
      return;
    }
    const bool whole = (e & (1u << 29)) && !tail;
    const int y = y0 + 16 * ty + l15;
    const bool y_in = y_all || (unsigned)y < (unsigned)n;
    float* ot = (STAGE ? st_o : orow) + 16 * ty;
    float* rt = rrow + 16 * ty;
    unsigned bits = 0;
    float be = 0.f;
    if (PREP) be = aux[16 * ty + l15];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int j = 16 * ty + l15 - 4 * zq - r;
      if (whole || (x0 + 4 * zq + r < n && j >= 0 && j < Wo)) {
        float v = y_in ? c[r] : 0.f;  // outside the matrix: the reference's zero fill
        if (PREP) {
          float rv = 0.f;
          if (y_in) {
            const float sh = al[r] + be;
            const bool ok = (v >= thr) && (v < INFINITY) && (sh > 0.9f * kFloor) && (sh < INFINITY);
            rv = ok ? __builtin_amdgcn_rcpf(v) : -1.f;  // -1 tells the backward that 1/S is not usable here
            v = __builtin_fmaf(fast_log2(v), kLn2, sh);
            if (!ok) bits |= 1u << r;
          }
          rt[ooff[r]] = rv;
        } else if (!(fabsf(v) <= FLT_MAX)) {
          redo = 1;
        }
        ot[ooff[r]] = v;
      }
    }
    if (PREP) redo |= (unsigned long long)bits << (4 * ty);
  };

  // ---- the walk: the loads of Q run kDirDepth steps ahead (past the end they repeat the
  // last step's and are never used); the words of the plan are read a step before their use
  const int steps = plan.steps;
  mm_f4 qraw[kDirDepth];
#pragma unroll
  for (int s = 0; s < kDirDepth; ++s) issue(plan.e[s].now, qraw[s]);
  mm_f4 c = mm_f4{0.f, 0.f, 0.f, 0.f};
  DirStep w = plan.e[0];
  for (int i = 0; i < steps; i += kDirDepth) {
#pragma unroll
    for (int s = 0; s < kDirDepth; ++s) {
      const DirStep cur = w;
      w = plan.e[i + s + 1];  // one entry past the last exists
      const unsigned e = cur.now;
      mask(e, qraw[s]);
      const mm_f4 qv = to_mfma(qraw[s]);
      const mm_f4 pv = pl[64 * ((e >> 12) & 7u)];
      issue(cur.ahead, qraw[s]);
      if (!(e & (1u << 27))) {  // uniform: not one of the filling steps
#pragma unroll
        for (int t = 0; t < 4; ++t) c = __builtin_amdgcn_mfma_f32_16x16x4f32(pv[t], qv[t], c, 0, 0, 0);
      }
      if (e & (1u << 19)) {  // uniform: the tile is complete
        finish(e, c);
        c = mm_f4{0.f, 0.f, 0.f, 0.f};
      }
    }
  }

  if (STAGE) {  // the tile row's 16 Wo results: one contiguous run of memory
    const mm_f4* so4 = reinterpret_cast<const mm_f4*>(st_o);
    for (int i = lane; i < 4 * Wo; i += 64) {
      const mm_f4 v = so4[i];
      *reinterpret_cast<dir_f4u*>(orow + 4 * i) = dir_f4u{v[0], v[1], v[2], v[3]};
    }
  }

  // ---- cells to recompute (rare).  The stores above are to the same addresses from the
  // same lane: they stay in order.
  if (!PREP && !(worst == 0.f)) redo = ~0ull;
  if (__builtin_amdgcn_ballot_w64(redo != 0) != 0) {
    if (!PREP && redo) redo = ~0ull;
    while (redo) {
      const int bit = __builtin_ctzll(redo);
      redo &= redo - 1;
      const int ty = bit >> 2, r = bit & 3;
      const int x = x0 + 4 * zq + r, j = 16 * ty + l15 - 4 * zq - r;
      if (ty < ny && x < n && j >= 0 && j < Wo) {
        if (PREP) band_fwd_cell<GENBMM_BAND_LOG>(p, bn + x, x, j);
        else band_fwd_cell<GENBMM_BAND_MUL>(p, bn + x, x, j);
      }
    }
  }
}

// One wave per tile row, kDirWaves tile rows per workgroup.  blocks: workgroups per batch item;
// wave_lds: bytes of LDS per wave.
template <bool PREP>
__global__ __launch_bounds__(64 * kDirWaves) void k_band_dir_fwd(const BandArgs p, const DirPlan plan, int blocks, int nblocks,
                                                     long cells_a, long cells_b, int wave_lds) {
  extern __shared__ __attribute__((aligned(16))) float dir_smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int blk = xcd_renumber(blockIdx.x, nblocks);
  const int batch = blk / blocks;
  const int x0 = ((blk - batch * blocks) * kDirWaves + wave) * 16;
  const int n = p.n, Wa = p.Wa, Wb = p.Wb;
  if (x0 >= n) return;
  const long bn = (long)batch * n;
  float* lds = dir_smem + wave * (wave_lds >> 2);
  // May the wave take 16-byte loads and skip the tests against the matrix?  Every band cell of
  // its rows of a inside the matrix (a cell of b that is not then only ever meets a zero), and
  // the cells that the loads can touch beside the band rows inside the tensors.
  const int ny = (p.Wo + 30) >> 4;
  const long y0 = bn + x0 - p.r_lu;
  const bool inside_matrix = x0 - p.a_lu >= 0 && x0 + 15 + (Wa - 1 - p.a_lu) <= n - 1;
  const bool inside_tensor = (bn + x0) * (long)Wa >= 16 && (bn + x0 + 15) * (long)Wa + 16 * kDirChunks + 4 <= cells_a &&
                             y0 * (long)Wb >= 16 * kDirChunks + 32 &&
                             (y0 + 16 * ny) * (long)Wb + 16 * kDirChunks + 32 <= cells_b;
  if (inside_matrix && inside_tensor) dir_fwd_row<PREP, false>(p, plan, bn, x0, lane, lds, cells_a, cells_b);
  else dir_fwd_row<PREP, true>(p, plan, bn, x0, lane, lds, cells_a, cells_b);
}

}  // namespace genbmm
