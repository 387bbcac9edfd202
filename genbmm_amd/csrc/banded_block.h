// Banded (+,*) products as block-banded matrix products on the matrix cores, operands staged
// through LDS as three bfloat16 parts (split_bf16.h): the plain product and the log product on
// the forward's workspace.
//
// A band tensor with rows of W cells is, read with a row pitch of W - 1, the dense matrix
// itself: cell c of band row r is the dense element (r, r + c - lu), and the dense element
// (r, q) lies at r (W - 1) + q + lu.  A 32 x 32 block of the dense matrix is therefore 32 runs
// of 32 neighbouring cells, one per band row - read as they lie, cells that belong to a
// neighbouring band row (outside [0, W) of this one) replaced by zeros.
//
//   forward   out[x, y] = sum_z A[x, z] B[y, z]      A[x, z] = a[x][z - x + lu_a], B[y, z] = b[y][z - y + lu_b]
//
// A workgroup walks down a run of 32-row blocks of one batch item ("steps").  A step multiplies
// the 32 rows x of A with the rows y of B its result band can meet: NT blocks of 32 rows y,
// each over the slabs (16 values of z) that both blocks' bands share.  Rows of B stay in LDS
// for as long as steps need them - a ring of NT + 1 blocks, every row of either operand read
// from memory and cut into its parts once.  One wave per block of a step multiplies and writes
// its 32 x 32 results from the accumulators; four more waves only stage, their loads two steps
// ahead of their use (two steps' worth of rows in flight per compute unit); all meet at one
// barrier per step.  (Ahead of the first step, which needs NT + 1 blocks staged, four of the
// multiplying waves stage half of them.)  The staging waves issue the same loads every step whatever the step meets
// - addresses are held inside the tensors, rows outside the matrix zeroed when they are staged -
// so that the counted waits for loads stay exact; a branch around a load costs every wait
// behind it its count.
//
// What bounds it (64 x 4096, 65 diagonals per operand: 73-78 us, of which the matrix instructions
// fill a tenth): instruction issue.  A step is about 900 staging instructions (cutting 6 144
// floats into parts), 220 matrix and LDS instructions and 500 for writing results, on four
// SIMDs that issue one vector instruction in about 4.4 cycles each; the staged blocks take 144
// of a compute unit's 160 KB of LDS, which is what keeps bands beyond 65 diagonals, a second
// workgroup per compute unit and a staging area for the results (wide contiguous stores) out.
//
// Staged form of a block: per slab three planes (the three parts) of [2 halves of the slab's z]
// [32 lines][4 words], a word holding two neighbouring z as bfloat16; a lane's operand of the
// matrix instruction is one 16-byte read, the 32 lanes of a half reading 512 bytes in a row.
//
// What is not finite in a result (an operand that is not, against a zero of the padding; a
// part that overflowed), and in the plain product an operand too small to be cut into parts
// exactly, is recomputed by the per-cell routine.
#pragma once

#include <cfloat>

#include "banded_flat.h"
#include "split_bf16.h"

namespace GENBMM_NS {

constexpr int kBlkNT = 6;                  // result blocks per step, at most
constexpr int kBlkOwn = 3;                 // result blocks per step and wave, at most
constexpr int kBlkSlabWords = 3 * 32 * 8;  // a slab of a 32-line block: three planes of [32 lines][8 words]
constexpr int kBlkPlaneWords = 32 * 8;
constexpr size_t kBlkLdsLimit = 160 * 1024;

struct BlkOwn {
  int t, lo, hi, off;  // block t: the first operand's slabs [lo, hi) with slabs sa - off of the second
};
struct BlkPlan {
  int NT;     // blocks of 32 result columns per step
  int NSa;    // slabs of a 32-row block of the first operand (z from x0 - lu_a)
  int NSb;    // slabs of a 32-row block of the second (z from y0 - lu_b - delta: on the first's grid)
  int delta;
  int chunk_steps, chunks;  // steps per workgroup, workgroups per batch item
  int ncw;                  // multiplying waves
  int count[kBlkNT];        // blocks of each
  BlkOwn own[kBlkNT][kBlkOwn];
};

// staged blocks, the row maxima of the log product (two steps of alpha, a ring of beta), a flag
inline size_t blk_lds_bytes(const BlkPlan& g) {
  return sizeof(unsigned) * ((size_t)kBlkSlabWords * (2 * g.NSa + (g.NT + 1) * g.NSb) + 32 * (2 + g.NT + 1) + 4);
}

// max_slabs: slabs per block that the kernel's register arrays take
inline bool blk_plan_fwd(BlkPlan& g, int Wa, int Wb, int n, int B, int max_slabs) {
  const int Wo = Wa + Wb - 1;
  g.NT = (31 + Wo + 31) / 32;
  g.NSa = (31 + Wa + 15) / 16;
  g.delta = (16 - (Wb - 1) % 16) % 16;
  g.NSb = (g.delta + 31 + Wb + 15) / 16;
  if (g.NT > kBlkNT || g.NSa > max_slabs || g.NSb > max_slabs) return false;
  if (blk_lds_bytes(g) > kBlkLdsLimit) return false;
  BlkOwn b[kBlkNT];
  for (int t = 0; t < g.NT; ++t) {
    b[t].t = t;
    b[t].off = 2 * t - (Wb - 1 + g.delta) / 16;
    // z - (x0 - lu_a) that both blocks' bands can hold: [0, 31 + Wa) and 32 t - (Wb - 1) + [0, 31 + Wb)
    const int plo = max(0, 32 * t - (Wb - 1)), phi = min(31 + Wa - 1, 32 * t + 31);
    b[t].lo = plo <= phi ? plo / 16 : 0;
    b[t].hi = plo <= phi ? phi / 16 + 1 : 0;
    if (b[t].hi > g.NSa || b[t].lo - b[t].off < 0 || (b[t].hi > b[t].lo && b[t].hi - 1 - b[t].off >= g.NSb)) return false;
  }
  for (int i = 0; i < g.NT; ++i)  // longest first, each to the wave with the least so far
    for (int j = i + 1; j < g.NT; ++j)
      if (b[j].hi - b[j].lo > b[i].hi - b[i].lo) { const BlkOwn x = b[i]; b[i] = b[j]; b[j] = x; }
  // A wave per block.  Wave w runs on SIMD w % 4, the staging waves (NT ... NT + 3) behind them:
  // the blocks in order of what they cost (instructions: a block with cells outside the result
  // band pays for testing every cell), dearest first, so that the SIMDs that take two get cheap ones.
  auto cost = [&](const BlkOwn& x) {
    const bool whole = 32 * x.t - 31 >= 0 && 32 * x.t + 31 < Wo;
    return 12 * (x.hi - x.lo) + (whole ? 120 : 250);
  };
  for (int i = 0; i < g.NT; ++i)
    for (int j = i + 1; j < g.NT; ++j)
      if (cost(b[j]) > cost(b[i])) { const BlkOwn x = b[i]; b[i] = b[j]; b[j] = x; }
  g.ncw = g.NT;
  for (int w = 0; w < g.NT; ++w) {
    g.count[w] = 1;
    g.own[w][0] = b[w];
  }
  // one workgroup per compute unit (LDS); about one round of workgroups over the chip
  const int steps = (n + 31) / 32;
  int chunks = max(1, min(steps, (256 + B - 1) / max(B, 1)));
  g.chunk_steps = (steps + chunks - 1) / chunks;
  g.chunks = (steps + g.chunk_steps - 1) / g.chunk_steps;
  return true;
}

// A piece (a line, four z) into the three planes at dst.  low: the lowest binary exponent seen so
// far among the values that are not zero (a value below 2^-100 does not come apart exactly).
template <bool CHECK>
__device__ __forceinline__ void blk_put(unsigned* __restrict__ dst, float4 v, int& low) {
  unsigned h0, m0, l0, h1, m1, l1;
  split2(v.x, v.y, h0, m0, l0);
  split2(v.z, v.w, h1, m1, l1);
  uintx2 w;
  w.x = h0; w.y = h1; *reinterpret_cast<uintx2*>(dst) = w;
  w.x = m0; w.y = m1; *reinterpret_cast<uintx2*>(dst + kBlkPlaneWords) = w;
  w.x = l0; w.y = l1; *reinterpret_cast<uintx2*>(dst + 2 * kBlkPlaneWords) = w;
  if (CHECK) {  // the exponent instruction gives 0 for a zero
    low = min(low, min(__builtin_amdgcn_frexp_expf(v.x), __builtin_amdgcn_frexp_expf(v.y)));
    low = min(low, min(__builtin_amdgcn_frexp_expf(v.z), __builtin_amdgcn_frexp_expf(v.w)));
  }
}
constexpr int kBlkLowExp = -99;

__device__ __forceinline__ float4 blk_and(float4 v, const unsigned (&m)[4]) {
  return make_float4(__uint_as_float(__float_as_uint(v.x) & m[0]), __uint_as_float(__float_as_uint(v.y) & m[1]),
                     __uint_as_float(__float_as_uint(v.z) & m[2]), __uint_as_float(__float_as_uint(v.w) & m[3]));
}

// the element at `bytes` from p
template <class E>
__device__ __forceinline__ const E* blk_at(const E* p, unsigned bytes) {
  return reinterpret_cast<const E*>(reinterpret_cast<const char*>(p) + bytes);
}
template <class E>
__device__ __forceinline__ E* blk_at(E* p, unsigned bytes) {
  return reinterpret_cast<E*>(reinterpret_cast<char*>(p) + bytes);
}
__device__ __forceinline__ bf16x8 blk_frag(const unsigned* q) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4*>(q));
}
// the six products of a slab; the two accumulators take them in turn
struct BlkFrags {
  bf16x8 ah, am, al, bh, bm, bl;
  __device__ __forceinline__ void read(const unsigned* a, const unsigned* b) {
    ah = blk_frag(a); bl = blk_frag(b + 2 * kBlkPlaneWords);
    al = blk_frag(a + 2 * kBlkPlaneWords); bh = blk_frag(b);
    bm = blk_frag(b + kBlkPlaneWords); am = blk_frag(a + kBlkPlaneWords);
  }
  // the two accumulators take the products in turn
  __device__ __forceinline__ void mul(floatx16& c0, floatx16& c1) const {
    c0 = mfma_bf16(ah, bl, c0);
    c1 = mfma_bf16(al, bh, c1);
    c0 = mfma_bf16(ah, bm, c0);
    c1 = mfma_bf16(am, bm, c1);
    c0 = mfma_bf16(am, bh, c0);
    c1 = mfma_bf16(ah, bh, c1);
  }
};

// SW: staging waves; a staging thread takes the slabs part, part + SW / 2, ... of a block (part: its
// wave pair), UA of the first and UB of the second operand's at most.
template <bool PREP, int SW, int UA, int UB>
__global__ __launch_bounds__(64 * (kBlkNT + SW)) void k_band_blk_fwd(const BandArgs p, const BlkPlan g, int nblocks,
                                                              long rows) {
  extern __shared__ __attribute__((aligned(16))) unsigned blk_smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int blk = xcd_renumber(blockIdx.x, nblocks);
  const int batch = blk / g.chunks, chunk = blk - batch * g.chunks;
  const int n = p.n, Wa = p.Wa, Wb = p.Wb, Wo = p.Wo;
  const int i_start = chunk * g.chunk_steps * 32;
  const int steps = min(g.chunk_steps, (n - i_start + 31) >> 5);
  if (steps <= 0) return;
  const long bn = (long)batch * n;
  const int NT = g.NT, NSa = g.NSa, NSb = g.NSb, RING = NT + 1;
  unsigned* const As = blk_smem;                                // two buffers of NSa slabs
  unsigned* const Bs = blk_smem + 2 * NSa * kBlkSlabWords;      // RING blocks of NSb slabs
  float* const alpha = reinterpret_cast<float*>(Bs + RING * NSb * kBlkSlabWords);  // [2][32]
  float* const beta = alpha + 64;                                                   // [RING][32]
  unsigned* const inexact = reinterpret_cast<unsigned*>(beta + 32 * RING);
  if (!PREP && tid == 0) *inexact = 0u;

  const int role = wave < g.ncw ? wave : wave - g.ncw;  // among the waves of its kind
  // ------------------------------------------------------------------ staging
  // The staging waves; the first four multiplying waves stage too, once: before the first step half
  // of the blocks that it needs are theirs (they would only wait for them).
  const bool helps = wave < g.ncw && wave < 4;
  constexpr int SP = SW / 2;
  const int lt = (wave < g.ncw ? wave & 3 : role) * 64 + lane, quad = lt & 3, line = (lt >> 2) & 31, half = lt >> 7;  // half: the wave pair
  auto asrc = [&] {
    if constexpr (PREP) return static_cast<const float*>(p.ws_ea);
    else return p.a;
  }();
  auto bsrc = [&] {
    if constexpr (PREP) return static_cast<const float*>(p.ws_eb);
    else return p.b;
  }();
  constexpr int ES = sizeof(*asrc);
  const long cells_a = rows * Wa, cells_b = rows * Wb;
  int low = 0;
  // What does not change from step to step: where a piece lies from its block's first cell
  // (a piece with no cell inside the band reads its row's first cells instead) and which of
  // its cells are inside the band.
  int offa[UA], offb[UB];
  unsigned ma[UA][4], mb[UB][4];
#pragma unroll
  for (int u = 0; u < UA; ++u) {
    const int slab = SP * u + half, c = 16 * slab + 4 * quad - line;
    offa[u] = line * Wa + (slab < NSa && c > -4 && c < Wa ? c : 0);
#pragma unroll
    for (int e = 0; e < 4; ++e) ma[u][e] = slab < NSa && (unsigned)(c + e) < (unsigned)Wa ? ~0u : 0u;
  }
#pragma unroll
  for (int u = 0; u < UB; ++u) {
    const int slab = SP * u + half, c = 16 * slab + 4 * quad - g.delta - line;
    offb[u] = line * Wb + (slab < NSb && c > -4 && c < Wb ? c : 0);
#pragma unroll
    for (int e = 0; e < 4; ++e) mb[u][e] = slab < NSb && (unsigned)(c + e) < (unsigned)Wb ? ~0u : 0u;
  }
  // a piece's place in a plane: [half of the slab's z][line][4 words], the lines of the second
  // half swapped in fours (the sixteen lanes that store together then meet sixteen banks)
  const int place = (quad >> 1) * 128 + ((line ^ ((quad >> 1) << 2)) << 2) + (quad & 1) * 2;
  unsigned* const dst_a = As + half * kBlkSlabWords + place;
  unsigned* const dst_b = Bs + half * kBlkSlabWords + place;

  // Every step issues the same loads whatever it meets (the waits then count exactly what is
  // in flight, two steps' worth): all of a block's pieces are read, from addresses held inside
  // the tensor.  A block's rows outside the matrix read their neighbours in memory and are
  // zeroed when they are staged; a piece that would cross an end of the tensor is read from
  // the four cells at that end and moved into place then.
  struct Where {
    long first;  // the cell of the tensor that offset 0 stands for
    int add;     // what a piece's offset from its block's first cell becomes an offset from `first` by
    int hi;      // the largest offset to read at
  };
  // (a piece may begin up to three cells ahead of its block's first cell)
  const long cell_a0 = (bn + i_start) * Wa, cell_b0 = (bn + i_start - p.r_lu) * Wb;  // first cells of block 0
  // the blocks of this workgroup (first operand: k, second: q) that lie clear of their tensor's ends
  auto clear_of_ends = [](long cell0, long per_block, long span, long cells, int& lo, int& hi) {
    lo = cell0 >= 4 ? 0 : (int)min((4 - cell0 + per_block - 1) / per_block, 1L << 30);
    const long room = cells - span - cell0;
    hi = room < 0 ? -1 : (int)min(room / per_block, 1L << 30);
  };
  int ka_lo, ka_hi, qb_lo, qb_hi;
  clear_of_ends(cell_a0, 32L * Wa, 31L * Wa + 16 * NSa + 8, cells_a, ka_lo, ka_hi);
  clear_of_ends(cell_b0, 32L * Wb, 31L * Wb + 16 * NSb + 8, cells_b, qb_lo, qb_hi);
  auto where = [&](long r0, long cells, bool clear) __attribute__((always_inline)) {
    Where w;
    if (clear) {  // uniform
      w.first = r0 - 4;
      w.add = 4;
      w.hi = 1 << 30;
    } else {
      w.first = min(max(r0 - 4, 0L), cells - 4);
      w.add = (int)min(max(r0 - w.first, -(1L << 30)), 1L << 30);
      w.hi = (int)min(cells - 4 - w.first, 1L << 30);
    }
    return w;
  };
  // a piece as it was meant, from what was read `shift` cells before it (cells that were not read: 0,
  // they lie outside the tensor)
  auto moved = [](float4 v, int shift) __attribute__((always_inline)) {
    const float x[4] = {v.x, v.y, v.z, v.w};
    float y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      y[e] = 0.f;
#pragma unroll
      for (int f = 0; f < 4; ++f) y[e] = f - e == shift ? x[f] : y[e];
    }
    return make_float4(y[0], y[1], y[2], y[3]);
  };
  // block k of the first operand: rows i_start + 32 k ..., z from i_start + 32 k - lu_a.
  // ab: alpha of the block's rows (lanes 0-31 of the first staging wave)
  auto load_a = [&](int k, float4 (&r)[UA], float& ab) __attribute__((always_inline)) {
    const int ib = i_start + 32 * k;
    const Where w = where(cell_a0 + 32 * k * Wa, cells_a, k >= ka_lo && k <= ka_hi);
    const auto* base = asrc + w.first;
#pragma unroll
    for (int u = 0; u < UA; ++u) r[u] = ld4(blk_at(base, (unsigned)(ES * min(max(offa[u] + w.add, 0), w.hi))));
    if (PREP) ab = p.ws_al[min(bn + ib + (lt & 31), rows - 1)];
  };
  // block q of the second: rows i_start - lu_out + 32 q ..., z from that - lu_b - delta.
  // ab: beta of the block's rows (lanes 32-63 of the first staging wave)
  auto load_b = [&](int q, float4 (&r)[UB], float& ab) __attribute__((always_inline)) {
    const int ob = i_start - p.r_lu + 32 * q;
    const Where w = where(cell_b0 + 32 * q * Wb, cells_b, q >= qb_lo && q <= qb_hi);
    const auto* base = bsrc + w.first;
#pragma unroll
    for (int u = 0; u < UB; ++u) r[u] = ld4(blk_at(base, (unsigned)(ES * min(max(offb[u] + w.add, 0), w.hi))));
    if (PREP) {
      const float be = p.ws_be[min(max(bn + ob + (lt & 31), 0L), rows - 1)];
      ab = lt & 32 ? be : ab;
    }
  };
  auto stage_a = [&](int k, const float4 (&r)[UA], float ab) __attribute__((always_inline)) {
    unsigned* dst = dst_a + (k & 1) * NSa * kBlkSlabWords;
    const int ib = i_start + 32 * k, z0 = ib - p.a_lu;
    const Where w = where(cell_a0 + 32 * k * Wa, cells_a, k >= ka_lo && k <= ka_hi);
    // uniform: every row of the block is a row of the matrix and every z of its slabs a column; no
    // piece had to be read elsewhere
    const bool plain = ib + 31 < n && z0 >= 0 && z0 + 16 * NSa <= n && w.add == 4 && w.hi >= 31 * Wa + 16 * NSa + 4;
#pragma unroll
    for (int u = 0; u < UA; ++u) {
      if (SP * u + half < NSa) {
        float4 v = r[u];
        if (!plain) {
          const int at = offa[u] + w.add;
          v = moved(v, at - min(max(at, 0), w.hi));
          const int z = z0 + 16 * (SP * u + half) + 4 * quad;
          const bool row = ib + line < n;
          v.x = row && (unsigned)(z + 0) < (unsigned)n ? v.x : 0.f;
          v.y = row && (unsigned)(z + 1) < (unsigned)n ? v.y : 0.f;
          v.z = row && (unsigned)(z + 2) < (unsigned)n ? v.z : 0.f;
          v.w = row && (unsigned)(z + 3) < (unsigned)n ? v.w : 0.f;
        }
        blk_put<!PREP>(dst + SP * u * kBlkSlabWords, blk_and(v, ma[u]), low);
      }
    }
    if (PREP && lt < 32) alpha[(k & 1) * 32 + lt] = ib + lt < n ? ab : 0.f;
  };
  auto stage_b = [&](int q, const float4 (&r)[UB], float ab) __attribute__((always_inline)) {
    const int slot = q % RING;
    unsigned* dst = dst_b + slot * NSb * kBlkSlabWords;
    const int ob = i_start - p.r_lu + 32 * q;
    const Where w = where(cell_b0 + 32 * q * Wb, cells_b, q >= qb_lo && q <= qb_hi);
    const bool plain = ob >= 0 && ob + 31 < n && w.add == 4 && w.hi >= 31 * Wb + 16 * NSb + 4;  // uniform
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      if (SP * u + half < NSb) {
        float4 v = r[u];
        if (!plain) {
          const int at = offb[u] + w.add;
          v = moved(v, at - min(max(at, 0), w.hi));
          const bool row = (unsigned)(ob + line) < (unsigned)n;
          v.x = row ? v.x : 0.f;
          v.y = row ? v.y : 0.f;
          v.z = row ? v.z : 0.f;
          v.w = row ? v.w : 0.f;
        }
        blk_put<!PREP>(dst + SP * u * kBlkSlabWords, blk_and(v, mb[u]), low);
      }
    }
    if (PREP && lt >= 32 && lt < 64) beta[slot * 32 + lt - 32] = (unsigned)(ob + lt - 32) < (unsigned)n ? ab : 0.f;
  };

  // of the NT - 1 older blocks of the second operand that step 0 meets, the first `helped` are staged by
  // the multiplying waves: half of the NT + 1 blocks to stage before the first step
  const int helped = g.ncw >= 4 ? min(NT - 1, (NT + 2) / 2) : 0;
  if (wave >= g.ncw) {
    float4 ra0[UA], rb0[UB], ra1[UA], rb1[UB];
    float aa0 = 0.f, aa1 = 0.f;  // alpha (lanes 0-31 of the first staging wave) or beta (its lanes 32-63)
    const int last = steps - 1;
    {
      // the blocks of the second operand that step 0 meets beside its own newest one
      // (blocks helped ... NT - 2 here, 0 ... helped - 1 by the multiplying waves that help)
      float4 pro[kBlkNT - 1][UB];
      float pab[kBlkNT - 1];
#pragma unroll
      for (int q = 0; q < kBlkNT - 1; ++q) {
        pab[q] = 0.f;
        load_b(min(helped + q, NT - 1), pro[q], pab[q]);
      }
      load_a(0, ra0, aa0);
      load_b(NT - 1, rb0, aa0);
      load_a(min(1, last), ra1, aa1);
      load_b(min(1, last) + NT - 1, rb1, aa1);
#pragma unroll
      for (int q = 0; q < kBlkNT - 1; ++q)
        if (helped + q < NT - 1) stage_b(helped + q, pro[q], pab[q]);
    }
    stage_a(0, ra0, aa0);
    stage_b(NT - 1, rb0, aa0);
    __syncthreads();
    // step s: ask for step s + 2, stage step s + 1 (asked for a step ago).  Past the last step the
    // loads repeat the last step's, and what is staged goes where no step looks any more - the
    // same instructions every time round, so that the waits for loads stay exact.
    int s = 0;
    for (; s + 1 < steps; s += 2) {
      load_a(min(s + 2, last), ra0, aa0);
      load_b(min(s + 2, last) + NT - 1, rb0, aa0);
      stage_a(s + 1, ra1, aa1);
      stage_b(s + NT, rb1, aa1);
      __syncthreads();
      load_a(min(s + 3, last), ra1, aa1);
      load_b(min(s + 3, last) + NT - 1, rb1, aa1);
      stage_a(s + 2, ra0, aa0);
      stage_b(s + 1 + NT, rb0, aa0);
      __syncthreads();
    }
    if (s < steps) __syncthreads();  // the last of an odd number of steps: nothing left to stage
    if (!PREP && low < kBlkLowExp) *inexact = 1u;
  } else {
    // ------------------------------------------------------------------ products
    // the multiplying waves are what a step waits for: they issue ahead of the staging waves
    __builtin_amdgcn_s_setprio(3);
    const int col = lane & 31, hi32 = lane >> 5;
    const int frag_off = hi32 * 128 + ((col ^ (hi32 << 2)) << 2);  // the lane's 16 bytes of a plane
    const float thr = fast_exp2(-kBandGuardBits);
    const int count = g.count[role];
    BlkOwn own[kBlkOwn];
#pragma unroll
    for (int k = 0; k < kBlkOwn; ++k) own[k] = g.own[role][min(k, max(count - 1, 0))];
    // element e of a block: row 8 (e / 4) + 4 hi32 + e % 4, column col; from the block's first
    // cell it lies at row (Wo - 1) + col cells
    // (in bytes of an element of the result)
    unsigned at[16];
#pragma unroll
    for (int e = 0; e < 16; ++e)
      at[e] = (unsigned)sizeof(elem_t) * (unsigned)((8 * (e >> 2) + 4 * hi32 + (e & 3)) * (Wo - 1) + col);
    // Opaque at each use: as a 32-bit offset beside a scalar base a store needs no address
    // arithmetic; left to the compiler the offsets are widened ahead of the loop and cost a
    // register pair and a 64-bit addition each.
    auto off32 = [](unsigned x) __attribute__((always_inline)) {
      asm volatile("" : "+v"(x));
      return x;
    };
    if (helps) {
      float4 pro[(kBlkNT + 1) / 2][UB];
      float pab[(kBlkNT + 1) / 2];
#pragma unroll
      for (int q = 0; q < (kBlkNT + 1) / 2; ++q) {
        pab[q] = 0.f;
        load_b(min(q, NT - 1), pro[q], pab[q]);
      }
#pragma unroll
      for (int q = 0; q < (kBlkNT + 1) / 2; ++q)
        if (q < helped) stage_b(q, pro[q], pab[q]);
    }
    __syncthreads();
    if (!PREP && low < kBlkLowExp) *inexact = 1u;  // (behind the barrier: thread 0 has cleared the flag)
    for (int s = 0; s < steps; ++s) {
      const int ib = i_start + 32 * s;

      const unsigned* const A = As + (s & 1) * NSa * kBlkSlabWords + frag_off;
#pragma unroll
      for (int k = 0; k < kBlkOwn; ++k) {
        if (k >= count) break;  // uniform
        const int t = own[k].t, lo = own[k].lo, hi = own[k].hi;
        const int slot = (s + t) % RING;
        floatx16 acc0, acc1;
#pragma unroll
        for (int e = 0; e < 16; ++e) acc0[e] = acc1[e] = 0.f;
        // the operands of the next slab are asked for ahead of the products of this one
        const unsigned* a = A + lo * kBlkSlabWords;
        const unsigned* b = Bs + slot * NSb * kBlkSlabWords + frag_off + (lo - own[k].off) * kBlkSlabWords;
        BlkFrags f0, f1;
        f0.read(a, b);
        for (int sa = lo; sa < hi; sa += 2) {
          const int nx = sa + 1 < hi ? kBlkSlabWords : 0;
          f1.read(a + nx, b + nx);
          __builtin_amdgcn_sched_barrier(0);
          f0.mul(acc0, acc1);
          __builtin_amdgcn_sched_barrier(0);
          if (sa + 1 >= hi) break;
          const int nx2 = sa + 2 < hi ? 2 * kBlkSlabWords : kBlkSlabWords;
          f0.read(a + nx2, b + nx2);
          __builtin_amdgcn_sched_barrier(0);
          f1.mul(acc0, acc1);
          __builtin_amdgcn_sched_barrier(0);
          a += 2 * kBlkSlabWords;
          b += 2 * kBlkSlabWords;
        }
        // band cell of element e: 32 t + col - (its row in the block)
        const bool whole = 32 * t - 31 >= 0 && 32 * t + 31 < Wo && ib + 31 < n;  // uniform
        const int o = ib - p.r_lu + 32 * t + col;
        const bool o_in = (unsigned)o < (unsigned)n;
        elem_t* const obase = p.o0 + ((bn + ib) * (long)Wo + 32 * t);  // uniform
        float* const rbase = PREP ? p.ws_r + ((bn + ib) * (long)Wo + 32 * t) : nullptr;
        const float be = PREP ? beta[slot * 32 + col] : 0.f;
        const float* const al = alpha + (s & 1) * 32 + 4 * hi32;
        unsigned redo = 0;
        float worst = 0.f;  // stays 0 while every result is finite
        auto emit = [&](auto whole_c) __attribute__((always_inline)) {
          constexpr bool WHOLE = decltype(whole_c)::value;
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int ro = 8 * (e >> 2) + 4 * hi32 + (e & 3);
            if (WHOLE || (ib + ro < n && (unsigned)(32 * t + col - ro) < (unsigned)Wo)) {
              float v = acc0[e] + acc1[e];
              if (PREP) {
                float rv = 0.f;
                if (o_in) {
                  const float sh = al[8 * (e >> 2) + (e & 3)] + be;
                  const bool ok = (v >= thr) && (v < INFINITY) && (sh >= kFloor) && (sh < INFINITY);
                  rv = ok ? __builtin_amdgcn_rcpf(v) : -1.f;  // -1 tells the backward that 1/S is not usable here
                  v = __builtin_fmaf(fast_log2(v), kLn2, sh);
                  if (!ok) redo |= 1u << e;
                } else {
                  v = 0.f;  // outside the matrix: the reference's zero fill
                }
                *blk_at(rbase, (unsigned)(4 / sizeof(elem_t)) * off32(at[e])) = rv;
              } else {
                worst = __builtin_fmaf(v, 0.f, worst);  // 0 * v is NaN exactly when v is not finite
              }
              *blk_at(obase, off32(at[e])) = to_elem<elem_t>(v);
            }
          }
        };
        if (whole) emit(std::true_type{});
        else emit(std::false_type{});
        if (!PREP && !(worst == 0.f)) redo = 0xffffu;
        while (redo) {  // rare; the stores above came from this lane: they stay in order
          const int e = __builtin_ctz(redo);
          redo &= redo - 1;
          const int ro = 8 * (e >> 2) + 4 * hi32 + (e & 3), j = 32 * t + col - ro;
          if (ib + ro < n && (unsigned)j < (unsigned)Wo) {
            if (PREP) band_fwd_cell<GENBMM_BAND_LOG>(p, bn + ib + ro, ib + ro, j);
            else band_fwd_cell<GENBMM_BAND_MUL>(p, bn + ib + ro, ib + ro, j);
          }
        }
      }
      __syncthreads();
    }
  }
  if (!PREP) {
    __syncthreads();
    if (*inexact) {  // rare: every cell of the workgroup's rows again, by the per-cell routine
      const int nrows = min(32 * steps, n - i_start);
      for (int c = tid; c < nrows * Wo; c += (int)blockDim.x) {
        const int r = c / Wo, j = c - r * Wo;
        band_fwd_cell<GENBMM_BAND_MUL>(p, bn + i_start + r, i_start + r, j);
      }
    }
  }
}

}  // namespace GENBMM_NS
