// Factored logbmm on the fp32 matrix cores, for problems whose tiles are all
// full: M, N (forward) resp. the output and reduction extents (backward) are
// multiples of 128 / 16 and every row is 16-byte aligned.  No bounds checks, no
// index arithmetic in the loop: each lane walks fixed pointers slab by slab.
//
// A workgroup of four waves (2x2) owns a 128x128 output tile; each wave keeps a
// 64x64 quarter as 2x2 accumulator blocks of v_mfma_f32_32x32x2_f32 (fp32 in,
// fp32 accumulate).  The reduction axis is consumed in slabs of 16 through two
// LDS buffers: while the matrix cores work on slab s, the global loads of slab
// s+1 are in flight; they are turned into exp(x - shift) and written to the
// other buffer before the single barrier of the iteration.
#pragma once

#include "common.h"

namespace genbmm {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// D(32x32) += A(32x2) * B(2x32).  Lane l supplies A[l % 32][l / 32] and
// B[l / 32][l % 32] and holds D[8*(i/4) + 4*(l/32) + i%4][l % 32] in element i.
__device__ __forceinline__ floatx16 mfma_32x32x2(float a, float b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ int mfma_row(int i, int lane) {
  return 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
}

constexpr int kMT = 128;        // tile edge
constexpr int kMS = 16;         // slab depth
constexpr int kMLD = kMT + 4;   // LDS row stride of a [slab][tile] buffer
constexpr float kMfmaGuardBits = 40.f;

// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.
// Renumber them so that every XCD works on one contiguous run of tiles (the 16
// tiles of a batch item share their operands).
__device__ __forceinline__ int xcd_tile_id() {
  const int w = blockIdx.x, n = gridDim.x;
  return (n & 7) == 0 ? (w & 7) * (n >> 3) + (w >> 3) : w;
}

__device__ __forceinline__ float exp_st(float d) { return fast_exp2(d * kLog2e); }

// 32 matrix-core steps over one staged slab: rows from R[q][0..128), columns
// from Cs[q][0..128).
__device__ __forceinline__ void mfma_slab(const float* __restrict__ R, const float* __restrict__ Cs,
                                          int wr0, int wc0, int lane, floatx16 (&acc)[2][2]) {
  const int lrow = lane & 31, lk = lane >> 5;
  const float* rp = R + lk * kMLD + wr0 + lrow;
  const float* cp = Cs + lk * kMLD + wc0 + lrow;
#pragma unroll
  for (int q = 0; q < kMS; q += 2) {
    const float a0 = rp[q * kMLD], a1 = rp[q * kMLD + 32];
    const float b0 = cp[q * kMLD], b1 = cp[q * kMLD + 32];
    acc[0][0] = mfma_32x32x2(a0, b0, acc[0][0]);
    acc[0][1] = mfma_32x32x2(a0, b1, acc[0][1]);
    acc[1][0] = mfma_32x32x2(a1, b0, acc[1][0]);
    acc[1][1] = mfma_32x32x2(a1, b1, acc[1][1]);
  }
}

// Store a float4 read along the reduction axis of an [out][red] tile into a
// [red][out] LDS buffer (transposing), and one read along the out axis of a
// [red][out] tile (straight).
__device__ __forceinline__ void lds_put_t(float* __restrict__ buf, int out, int red4, float4 v) {
  float* p = buf + (red4 * 4) * kMLD + out;
  p[0] = v.x; p[kMLD] = v.y; p[2 * kMLD] = v.z; p[3 * kMLD] = v.w;
}
__device__ __forceinline__ void lds_put(float* __restrict__ buf, int red, int out4, float4 v) {
  *reinterpret_cast<float4*>(buf + red * kMLD + out4 * 4) = v;
}

// ----------------------------------------------------------------- forward
__global__ __launch_bounds__(256, 4) void k_log_fwd_mfma(const float* __restrict__ a,
                                                         const float* __restrict__ b,
                                                         float* __restrict__ out,
                                                         const float* __restrict__ stats,
                                                         int* __restrict__ flags, int M, int K,
                                                         int N, int tiles_m, int tiles_n) {
  __shared__ __attribute__((aligned(16))) float As[2][kMS * kMLD];
  __shared__ __attribute__((aligned(16))) float Bs[2][kMS * kMLD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
  const int per = tiles_m * tiles_n, tile = xcd_tile_id();
  const int batch = tile / per, rem = tile - batch * per;
  const int m0 = (rem / tiles_n) * kMT, n0 = (rem % tiles_n) * kMT;
  const float* st = stats + (long)batch * (M + N);

  // a tile [m][k]: lane reads rows ar, ar+64 at k quad aq;  b tile [k][n]: rows br, br+8
  const int ar = tid >> 2, aq = tid & 3, br = tid >> 5, bq = tid & 31;
  const float* pa = a + ((long)batch * M + m0 + ar) * K + aq * 4;
  const float* pb = b + ((long)batch * K + br) * N + n0 + bq * 4;
  const float al0 = st[m0 + ar], al1 = st[m0 + ar + 64];
  const float4 be = *reinterpret_cast<const float4*>(st + M + n0 + bq * 4);

  floatx16 acc[2][2];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[x >> 1][x & 1][i] = 0.f;

  float4 ra0, ra1, rb0, rb1;
  auto load = [&]() __attribute__((always_inline)) {
    ra0 = *reinterpret_cast<const float4*>(pa);
    ra1 = *reinterpret_cast<const float4*>(pa + 64l * K);
    rb0 = *reinterpret_cast<const float4*>(pb);
    rb1 = *reinterpret_cast<const float4*>(pb + 8l * N);
    pa += kMS;
    pb += (long)kMS * N;
  };
  auto stage = [&](int buf) __attribute__((always_inline)) {
    lds_put_t(As[buf], ar, aq, make_float4(exp_st(ra0.x - al0), exp_st(ra0.y - al0),
                                           exp_st(ra0.z - al0), exp_st(ra0.w - al0)));
    lds_put_t(As[buf], ar + 64, aq, make_float4(exp_st(ra1.x - al1), exp_st(ra1.y - al1),
                                                exp_st(ra1.z - al1), exp_st(ra1.w - al1)));
    lds_put(Bs[buf], br, bq, make_float4(exp_st(rb0.x - be.x), exp_st(rb0.y - be.y),
                                         exp_st(rb0.z - be.z), exp_st(rb0.w - be.w)));
    lds_put(Bs[buf], br + 8, bq, make_float4(exp_st(rb1.x - be.x), exp_st(rb1.y - be.y),
                                             exp_st(rb1.z - be.z), exp_st(rb1.w - be.w)));
  };

  const int slabs = K / kMS;
  load();
  stage(0);
  __syncthreads();
  for (int s = 0; s < slabs; ++s) {
    const bool more = s + 1 < slabs;
    if (more) load();
    mfma_slab(As[s & 1], Bs[s & 1], wm0, wn0, lane, acc);
    if (more) stage((s + 1) & 1);
    __syncthreads();
  }

  // guard: S >= 2^-40, finite, and the shift above the reference's -1e9 floor
  const float thr = fast_exp2(-kMfmaGuardBits);
  const int lrow = lane & 31;
  int bad = 0;
  float be_c[2];
  be_c[0] = st[M + n0 + wn0 + lrow];
  be_c[1] = st[M + n0 + wn0 + 32 + lrow];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float shift = st[m0 + wm0 + (x >> 1) * 32 + mfma_row(i, lane)] + be_c[x & 1];
      const float s = acc[x >> 1][x & 1][i];
      if (!((s >= thr) && (s < INFINITY) && (shift > 0.9f * kFloor) && (shift < INFINITY))) bad = 1;
      acc[x >> 1][x & 1][i] = __builtin_fmaf(fast_log2(s), kLn2, shift);
    }
  bad = __syncthreads_or(bad);
  if (tid == 0) flags[tile] = bad;
  if (bad) return;  // the fix-up launch recomputes this tile
  float* ob = out + ((long)batch * M + m0 + wm0) * N + n0 + wn0 + lrow;
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i)
      ob[(long)((x >> 1) * 32 + mfma_row(i, lane)) * N + (x & 1) * 32] = acc[x >> 1][x & 1][i];
}

// ---------------------------------------------------------------- backward
// GRAD_A: tile (m,k) of grad_a, reduction over n.  rows <- H[n][m], cols <- EB[n][k].
// GRAD_B: tile (k,n) of grad_b, reduction over m.  rows <- EA[m][k], cols <- H[m][n].
// H = g * exp(alpha[m] + beta[n] - out[m,n]);  the epilogue multiplies by
// exp(x - shift) of the operand shaped like the output.
template <bool GRAD_A>
__global__ __launch_bounds__(256, GRAD_A ? 2 : 4) void k_log_bwd_mfma(const float* __restrict__ a,
                                                         const float* __restrict__ b,
                                                         const float* __restrict__ outp,
                                                         const float* __restrict__ g,
                                                         const float* __restrict__ stats,
                                                         float* __restrict__ grad,
                                                         int* __restrict__ flags, int M, int K,
                                                         int N, int tiles_r, int tiles_c) {
  __shared__ __attribute__((aligned(16))) float Ys[2][kMS * kMLD];
  __shared__ __attribute__((aligned(16))) float Hs[2][kMS * kMLD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr0 = (wave >> 1) * 64, wc0 = (wave & 1) * 64;
  const int per = tiles_r * tiles_c, tile = xcd_tile_id();
  const int batch = tile / per, rem = tile - batch * per;
  const int r0 = (rem / tiles_c) * kMT, c0 = (rem % tiles_c) * kMT;
  const int Q = GRAD_A ? N : M;
  const float* al = stats + (long)batch * (M + N);
  const float* be = al + M;
  const float lim = kMfmaGuardBits * kLn2 + 1e-3f;

  floatx16 acc[2][2];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[x >> 1][x & 1][i] = 0.f;

  float4 ry0, ry1, ro0, ro1, rg0, rg1, sh;   // sh: shifts that change with the slab
  float sh0 = 0.f, sh1 = 0.f;
  int bad = 0;
  const float* py;
  const float* po;
  const float* pg;
  const float* ps;
  // fixed shifts
  float fa0 = 0.f, fa1 = 0.f;
  float4 fb = make_float4(0.f, 0.f, 0.f, 0.f);
  const int tr = tid >> 2, tq = tid & 3;    // [out][red] tiles: out row tr (+64), red quad tq
  const int ur = tid >> 5, uq = tid & 31;   // [red][out] tiles: red row ur (+8), out quad uq
  if constexpr (GRAD_A) {
    py = b + ((long)batch * K + c0 + tr) * N + tq * 4;      // b[k = c0+tr][n]
    po = outp + ((long)batch * M + r0 + tr) * N + tq * 4;   // out[m = r0+tr][n]
    pg = g + ((long)batch * M + r0 + tr) * N + tq * 4;
    ps = be + tq * 4;                                       // beta[n] of the slab
    fa0 = al[r0 + tr];
    fa1 = al[r0 + tr + 64];
  } else {
    py = a + ((long)batch * M + ur) * K + r0 + uq * 4;      // a[m][k = r0 + ...]
    po = outp + ((long)batch * M + ur) * N + c0 + uq * 4;   // out[m][n = c0 + ...]
    pg = g + ((long)batch * M + ur) * N + c0 + uq * 4;
    ps = al + ur;                                           // alpha[m] of the slab
    fb = *reinterpret_cast<const float4*>(be + c0 + uq * 4);
  }
  auto load = [&]() __attribute__((always_inline)) {
    if constexpr (GRAD_A) {
      ry0 = *reinterpret_cast<const float4*>(py);
      ry1 = *reinterpret_cast<const float4*>(py + 64l * N);
      ro0 = *reinterpret_cast<const float4*>(po);
      ro1 = *reinterpret_cast<const float4*>(po + 64l * N);
      rg0 = *reinterpret_cast<const float4*>(pg);
      rg1 = *reinterpret_cast<const float4*>(pg + 64l * N);
      sh = *reinterpret_cast<const float4*>(ps);
      py += kMS; po += kMS; pg += kMS; ps += kMS;
    } else {
      ry0 = *reinterpret_cast<const float4*>(py);
      ry1 = *reinterpret_cast<const float4*>(py + 8l * K);
      ro0 = *reinterpret_cast<const float4*>(po);
      ro1 = *reinterpret_cast<const float4*>(po + 8l * N);
      rg0 = *reinterpret_cast<const float4*>(pg);
      rg1 = *reinterpret_cast<const float4*>(pg + 8l * N);
      sh0 = ps[0];
      sh1 = ps[8];
      py += (long)kMS * K; po += (long)kMS * N; pg += (long)kMS * N; ps += kMS;
    }
  };
  auto hval = [&](float gv, float e) __attribute__((always_inline)) {
    if (!(e <= lim)) bad = 1;  // S < 2^-40 (or NaN): factoring not exact here
    return gv * exp_st(e);
  };
  auto stage = [&](int buf) __attribute__((always_inline)) {
    if constexpr (GRAD_A) {
      lds_put_t(Ys[buf], tr, tq, make_float4(exp_st(ry0.x - sh.x), exp_st(ry0.y - sh.y),
                                             exp_st(ry0.z - sh.z), exp_st(ry0.w - sh.w)));
      lds_put_t(Ys[buf], tr + 64, tq, make_float4(exp_st(ry1.x - sh.x), exp_st(ry1.y - sh.y),
                                                  exp_st(ry1.z - sh.z), exp_st(ry1.w - sh.w)));
      lds_put_t(Hs[buf], tr, tq,
                make_float4(hval(rg0.x, fa0 + sh.x - ro0.x), hval(rg0.y, fa0 + sh.y - ro0.y),
                            hval(rg0.z, fa0 + sh.z - ro0.z), hval(rg0.w, fa0 + sh.w - ro0.w)));
      lds_put_t(Hs[buf], tr + 64, tq,
                make_float4(hval(rg1.x, fa1 + sh.x - ro1.x), hval(rg1.y, fa1 + sh.y - ro1.y),
                            hval(rg1.z, fa1 + sh.z - ro1.z), hval(rg1.w, fa1 + sh.w - ro1.w)));
    } else {
      lds_put(Ys[buf], ur, uq, make_float4(exp_st(ry0.x - sh0), exp_st(ry0.y - sh0),
                                           exp_st(ry0.z - sh0), exp_st(ry0.w - sh0)));
      lds_put(Ys[buf], ur + 8, uq, make_float4(exp_st(ry1.x - sh1), exp_st(ry1.y - sh1),
                                               exp_st(ry1.z - sh1), exp_st(ry1.w - sh1)));
      lds_put(Hs[buf], ur, uq,
              make_float4(hval(rg0.x, sh0 + fb.x - ro0.x), hval(rg0.y, sh0 + fb.y - ro0.y),
                          hval(rg0.z, sh0 + fb.z - ro0.z), hval(rg0.w, sh0 + fb.w - ro0.w)));
      lds_put(Hs[buf], ur + 8, uq,
              make_float4(hval(rg1.x, sh1 + fb.x - ro1.x), hval(rg1.y, sh1 + fb.y - ro1.y),
                          hval(rg1.z, sh1 + fb.z - ro1.z), hval(rg1.w, sh1 + fb.w - ro1.w)));
    }
  };

  const int slabs = Q / kMS;
  load();
  stage(0);
  __syncthreads();
  for (int s = 0; s < slabs; ++s) {
    const bool more = s + 1 < slabs;
    if (more) load();
    if constexpr (GRAD_A)
      mfma_slab(Hs[s & 1], Ys[s & 1], wr0, wc0, lane, acc);
    else
      mfma_slab(Ys[s & 1], Hs[s & 1], wr0, wc0, lane, acc);
    if (more) stage((s + 1) & 1);
    __syncthreads();
  }

  bad = __syncthreads_or(bad);
  if (tid == 0) flags[tile] = bad;
  if (bad) return;  // the fix-up launch recomputes this tile

  // grad = exp(x - shift) * acc
  const int Cc = GRAD_A ? K : N;
  const int lrow = lane & 31;
  const float* xb = (GRAD_A ? a : b) + ((long)batch * (GRAD_A ? M : K) + r0 + wr0) * Cc + c0 + wc0 + lrow;
  float* gp = grad + ((long)batch * (GRAD_A ? M : K) + r0 + wr0) * Cc + c0 + wc0 + lrow;
  float cs[2] = {0.f, 0.f};
  if constexpr (!GRAD_A) {
    cs[0] = be[c0 + wc0 + lrow];
    cs[1] = be[c0 + wc0 + 32 + lrow];
  }
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int rr = (x >> 1) * 32 + mfma_row(i, lane);
      const long off = (long)rr * Cc + (x & 1) * 32;
      const float shv = GRAD_A ? al[r0 + wr0 + rr] : cs[x & 1];
      gp[off] = exp_st(xb[off] - shv) * acc[x >> 1][x & 1][i];
    }
}

}  // namespace genbmm
