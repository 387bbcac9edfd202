// logbmm for 32 x 32 x 32 items (the skinny chain shape): one wave per batch item, the
// contraction on v_mfma_f32_32x32x2_f32, no barrier and no operand tile in LDS.
//
// Same factored form as logbmm_item.h.  The instruction sums over two values of the
// contraction index per step, one from each half of the wave; which value a half feeds
// in which of the 16 steps is free as long as both operands agree.  Two such orders are
// used, each chosen so that an operand comes from memory already in the lane and register
// that feeds it:
//
//   * "rows": lane (i, h) holds x[i][16 h + s] in register s - its 16 values are 64
//     contiguous bytes of row i;
//   * "columns": lane (c, h) holds x[rho(r, h)][c] in register r, rho = 8 (r / 4) + 4 h + r % 4
//     - the rows the instruction's result leaves in that lane, so a product's result, the
//     factor it is multiplied by on the way out and the operand of the next product line up
//     register for register, and every load and store is 128 contiguous bytes per row.
//
// forward:  S[i][j] = sum_k EA[i][k] EB[k][j]      EA in rows, EB in columns (k = 16 h + s)
// grad_a:   T[i][k] = sum_j H[i][j] EB[k][j]       H in rows, EB in rows (j = 16 h + s): both are
//           computed in columns for grad_b and turned through LDS (the 16-byte loads of the
//           rows layout, one row per lane, cost the memory pipeline four times the columns');
//           T leaves in columns, where EA is read for grad_a = EA .* T
// grad_b:   U[k][j] = sum_i EA[i][k] H[i][j]       EA and H in columns (i = rho(r, h));
//           U leaves in columns, where EB is read for grad_b = EB .* U
//
// The maxima alpha, beta are taken in the wave (16 values per lane and one exchange between
// the halves) and passed through 64 floats of LDS to the lanes that need them by row.
// Cells (forward) or items (backward) for which the factoring is not exact to fp32 are
// recomputed from global memory with the reference's own form, as in logbmm_item.h.
#pragma once

#include "logbmm_item.h"
#include "logbmm_mfma.h"

namespace GENBMM_NS {

constexpr int kI32 = 32;  // M = K = N

struct Item32Lane {
  int c, h;  // lane & 31, lane >> 5
};

// 16 values x[row][16 h + s] of a row-major 32 x 32 item
__device__ __forceinline__ void item32_rows(const elem_t* __restrict__ x, int row, int h, float (&v)[16]) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float4 t = ld4(x + row * kI32 + 16 * h + 4 * q);
    v[4 * q] = t.x; v[4 * q + 1] = t.y; v[4 * q + 2] = t.z; v[4 * q + 3] = t.w;
  }
}
// 16 values x[k][c] for k = 16 h + s
__device__ __forceinline__ void item32_cols_k(const elem_t* __restrict__ x, int c, int h, float (&v)[16]) {
#pragma unroll
  for (int s = 0; s < 16; ++s) v[s] = x[(16 * h + s) * kI32 + c];
}
// 16 values x[rho(r, h)][c]
__device__ __forceinline__ void item32_cols(const elem_t* __restrict__ x, int c, int h, float (&v)[16]) {
#pragma unroll
  for (int r = 0; r < 16; ++r) v[r] = x[(mfma_row_u(r) + 4 * h) * kI32 + c];
}
__device__ __forceinline__ float max16(const float (&v)[16]) {
  float m = v[0];
#pragma unroll
  for (int s = 1; s < 16; ++s) m = fmaxf(m, v[s]);
  return fmaxf(m, __shfl_xor(m, 32, 64));  // the other half's 16
}

// One wave per item, four items per workgroup.
__global__ __launch_bounds__(256) void k_log_item32_fwd(const elem_t* __restrict__ a, const elem_t* __restrict__ b,
                                                       elem_t* __restrict__ out, float* __restrict__ stats,
                                                       int* __restrict__ hdr, int B) {
  __shared__ float sh[4][64];
  if (hdr && blockIdx.x == 0 && threadIdx.x == 0) hdr[0] = kWsNone;  // no per-tile flags in this workspace
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int item = blockIdx.x * 4 + wave;
  if (item >= B) return;
  const int c = lane & 31, h = lane >> 5;
  const elem_t* ab = a + (long)item * kI32 * kI32;
  const elem_t* bb = b + (long)item * kI32 * kI32;
  float av[16], bv[16];
  item32_rows(ab, c, h, av);      // a[i = c][16 h + s]
  item32_cols_k(bb, c, h, bv);    // b[16 h + s][j = c]
  const float al = max16(av), be = max16(bv);
  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
  for (int s = 0; s < 16; ++s) acc = mfma_32x32x2(item_exp(av[s], al), item_exp(bv[s], be), acc);
  // alpha of the rows this lane's results belong to
  float* shw = sh[wave];
  if (h == 0) shw[c] = al;
  wave_lds_sync();
  float ar[16];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float4 t = *reinterpret_cast<const float4*>(shw + 8 * q + 4 * h);
    ar[4 * q] = t.x; ar[4 * q + 1] = t.y; ar[4 * q + 2] = t.z; ar[4 * q + 3] = t.w;
  }
  if (stats) {
    float* st = stats + (long)item * 2 * kI32;
    st[lane] = h == 0 ? al : be;  // alpha[0..32), beta[0..32)
  }
  const float thr = fast_exp2(-kItemGuardBits);
  elem_t* ob = out + (long)item * kI32 * kI32;
  unsigned redo = 0;  // bit r: the cell is recomputed by the reference's form (rare)
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int i = mfma_row_u(r) + 4 * h;
    const float shift = ar[r] + be, s = acc[r];
    const bool ok = (s >= thr) && (s < INFINITY) && (shift >= kFloor) && (shift < INFINITY);
    if (!ok) redo |= 1u << r;
    ob[i * kI32 + c] = to_elem<elem_t>(__builtin_fmaf(fast_log2(s), kLn2, shift));
  }
  while (redo) {  // same lane, same address as the store above: they stay in order
    const int r = __builtin_ctz(redo);
    redo &= redo - 1;
    const int i = 8 * (r >> 2) + (r & 3) + 4 * h;
    ob[i * kI32 + c] = to_elem<elem_t>(item_exact_out(ab + i * kI32, bb + c, kI32, kI32));
  }
}

__global__ __launch_bounds__(256, 3) void k_log_item32_bwd(const elem_t* __restrict__ a, const elem_t* __restrict__ b,
                                                       const elem_t* __restrict__ outp, const elem_t* __restrict__ g,
                                                       elem_t* __restrict__ grad_a, elem_t* __restrict__ grad_b,
                                                       int B) {
  __shared__ float sh[4][64];
  __shared__ float tr[4][kI32 * 33];  // a wave's 32 x 32 values on their way from columns to rows
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int item = blockIdx.x * 4 + wave;
  if (item >= B) return;
  const int c = lane & 31, h = lane >> 5;
  constexpr int E = kI32 * kI32;
  float* tw = tr[wave];
  // x in columns (x[rho(r, h)][c] in register r)  ->  x in rows (x[c][16 h + s] in register s)
  auto to_rows = [&](const float (&col)[16], float (&row)[16]) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 16; ++r) tw[(mfma_row_u(r) + 4 * h) * 33 + c] = col[r];
    wave_lds_sync();
#pragma unroll
    for (int s2 = 0; s2 < 16; ++s2) row[s2] = tw[c * 33 + 16 * h + s2];
    wave_lds_sync();
  };
  const elem_t* ab = a + (long)item * E;
  const elem_t* bb = b + (long)item * E;
  const elem_t* ob = outp + (long)item * E;
  const elem_t* gb = g + (long)item * E;
  elem_t* gab = grad_a ? grad_a + (long)item * E : nullptr;
  elem_t* gbb = grad_b ? grad_b + (long)item * E : nullptr;

  // ---- everything the item needs is requested at once (one trip to memory, not one per phase)
  float a_col[16], b_col[16], g_col[16], o_col[16], al, be;
  {
    float a_row[16];
    item32_rows(ab, c, h, a_row);
    item32_cols(bb, c, h, b_col);   // b[rho][j = c]
    item32_cols(gb, c, h, g_col);
    item32_cols(ob, c, h, o_col);
    item32_cols(ab, c, h, a_col);   // a[rho][k = c]: the second read of a comes from the cache
    __builtin_amdgcn_sched_barrier(0);
    // ---- maxima: alpha from a in rows, beta from b in columns; both to LDS
    al = max16(a_row);  // alpha[c]
  }
  be = max16(b_col);              // beta[c]
  float* shw = sh[wave];
  if (h == 0) shw[c] = al;
  wave_lds_sync();
  float al_rho[16];  // alpha[rho(r, h)]
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float4 t = *reinterpret_cast<const float4*>(shw + 8 * q + 4 * h);
    al_rho[4 * q] = t.x; al_rho[4 * q + 1] = t.y; al_rho[4 * q + 2] = t.z; al_rho[4 * q + 3] = t.w;
  }

  // ---- H in columns, and whether the factoring is exact for this item
  float h_col[16];
  const float lim = kItemGuardBits * kLn2 + 1e-3f;
  int bad = 0;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float ex = al_rho[r] + be - o_col[r];
    if (!(ex <= lim) || !(ex > -INFINITY)) bad = 1;  // S < 2^-40, NaN or infinities: not exact
    h_col[r] = g_col[r] * fast_exp2(ex * kLog2e);
  }
  if (__builtin_amdgcn_ballot_w64(bad != 0) != 0) {
    // the reference's form for the whole item (matmul_cuda_kernel.cu:159-184):
    // exp(a + b - out) * g summed over n (grad_a) / m (grad_b), from global memory
    if (gab)
      for (int e = lane; e < E; e += 64) {
        const int m = e / kI32, k = e - m * kI32;
        const float av = ab[e];
        float s = 0.f;
        for (int n = 0; n < kI32; ++n)
          s = __builtin_fmaf(fast_exp(av + (float)bb[k * kI32 + n] - (float)ob[m * kI32 + n]), (float)gb[m * kI32 + n], s);
        gab[e] = to_elem<elem_t>(s);
      }
    if (gbb)
      for (int e = lane; e < E; e += 64) {
        const int k = e / kI32, n = e - k * kI32;
        const float bv = bb[e];
        float s = 0.f;
        for (int m = 0; m < kI32; ++m)
          s = __builtin_fmaf(fast_exp((float)ab[m * kI32 + k] + bv - (float)ob[m * kI32 + n]), (float)gb[m * kI32 + n], s);
        gbb[e] = to_elem<elem_t>(s);
      }
    return;
  }

  // ---- EA in columns: the factor of grad_a and the first operand of grad_b
#pragma unroll
  for (int r = 0; r < 16; ++r) a_col[r] = item_exp(a_col[r], al_rho[r]);

  // EB in columns: the factor of grad_b and, turned into rows, the second operand of grad_a
#pragma unroll
  for (int r = 0; r < 16; ++r) b_col[r] = item_exp(b_col[r], be);
  if (gbb) {  // U[k][j] = sum_i EA[i][k] H[i][j], i = rho(r, h): both operands in columns
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc = mfma_32x32x2(a_col[r], h_col[r], acc);
#pragma unroll
    for (int r = 0; r < 16; ++r) gbb[(mfma_row_u(r) + 4 * h) * kI32 + c] = to_elem<elem_t>((b_col[r] * acc[r]));
  }
  if (gab) {  // T[i][k] = sum_j H[i][j] EB[k][j], j = 16 h + s: both operands in rows
    float h_row[16], eb_row[16];
    to_rows(h_col, h_row);    // H[i = c][16 h + s]
    to_rows(b_col, eb_row);   // EB[k = c][16 h + s]
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
    for (int s2 = 0; s2 < 16; ++s2) acc = mfma_32x32x2(h_row[s2], eb_row[s2], acc);
#pragma unroll
    for (int r = 0; r < 16; ++r) gab[(mfma_row_u(r) + 4 * h) * kI32 + c] = to_elem<elem_t>((a_col[r] * acc[r]));
  }
}

}  // namespace GENBMM_NS
