// Double-precision logbmm on the matrix cores (v_mfma_f64_16x16x4_f64): forward, grad_a
// and grad_b in the factored form of the float path, with no workspace.
//
//   alpha[m] = max_k a[m,k], beta[n] = max_k b[k,n], EA = exp(a - alpha), EB = exp(b - beta)
//   S = EA EB,  out = log S + alpha + beta,  H = g / S = g exp(alpha + beta - out)
//   grad_a = EA .* (H EB^T),  grad_b = EB .* (EA^T H)
//
// so that (M K + K N + M N) exponentials replace the M K N of the reference's loops
// (matmul_cuda_kernel.cu:27-41, 159-217), and the contraction is a plain product.  All
// three are C[i,j] = sum_l P[i,l] Q[l,j] on 128 x 128 (or 64 x 64) tiles of (i,j), one
// workgroup of eight (four) waves per tile (each wave 32 x 64 or 32 x 32 of it: eight or four
// 16 x 16 accumulators), the contraction in chunks of 16 staged in LDS with the exponential taken
// on the way in; the next chunk's operands are in flight while the current one is
// multiplied.  The exponentials of a staged chunk are vector work of about the same cost as
// the chunk's matrix instructions at 64 x 64 and half of it at 128 x 128.
//
// The entry points have no workspace to keep the maxima in, so a workgroup takes them itself
// before its tile: the forward for its own rows and columns, grad_a for its rows and
// every column of the item, grad_b for every row and its columns (a pass over a and b that
// the L2 serves; a few percent of the tile's work up to a few hundred rows).
//
// Exact wherever the factors lose nothing: a sum S below 1e-280 (terms that underflow in the
// factored form could matter), a shift at the reference's -1e9 floor or anything not finite
// sends the cell to the reference's own loops (a forward cell: two passes over k; a
// gradient cell: the sum of exp(a + b - out) g), inside the same kernel.  H is NaN where S
// is not usable, which carries the flag through the product to every cell it feeds.
#pragma once

#include "common.h"

namespace GENBMM_NS {

constexpr int kDC = 16;        // contraction chunk
constexpr int kDP = kDC + 1;   // row pitch of a staged chunk, in doubles: odd, so that lanes four rows apart
                               // (the staging stores of an operand whose rows run along the reduction) and
                               // lanes one row apart (everything else) both spread over all LDS banks
constexpr double kDFloor = -1e9;
constexpr double kDThr = 1e-280;
constexpr double kDLogThr = -644.7;  // log(kDThr), rounded up

// exp for the factors (one per staged element: what these kernels spend their vector time on).
// The arguments are shifted operands (<= 0) and -log S (guarded to <= 645): finite results
// only, so no overflow handling; anything below -800 gives 0 and NaN stays NaN.  Reduction by
// ln 2 in two parts (the high part has 21 trailing zero bits, so n * hi is exact), Taylor
// polynomial of degree 13 on |r| <= 0.347 (truncation 4e-18), scaling by v_ldexp_f64:
// about 20 instructions against the 80 of the library routine, within 2 ulp of it.
// The coefficients live in constant memory and are not `const`: the compiler then reads them
// with scalar loads into scalar registers, where v_fma_f64 takes them as its addend.  As
// literals every one of them costs a 64-bit move per use (the instruction has no room for a
// 64-bit immediate), which doubles the polynomial.
__constant__ double d64_exp_c[16] = {1.0 / 6227020800.0, 1.0 / 479001600.0, 1.0 / 39916800.0, 1.0 / 3628800.0,
                                     1.0 / 362880.0,     1.0 / 40320.0,     1.0 / 5040.0,     1.0 / 720.0,
                                     1.0 / 120.0,        1.0 / 24.0,        1.0 / 6.0,        0.5,
                                     1.44269504088896340736, -6.93147180369123816490e-01,
                                     -1.90821492927058770002e-10, -800.0};
__device__ __forceinline__ double d64_exp(double x) {
  const double* c = d64_exp_c;
  x = x < c[15] ? c[15] : x;
  const double n = __builtin_rint(x * c[12]);
  double r = __builtin_fma(n, c[13], x);
  r = __builtin_fma(n, c[14], r);
  double p = c[0];
#pragma unroll
  for (int i = 1; i < 12; ++i) p = __builtin_fma(p, r, c[i]);
  p = __builtin_fma(p, r, 1.0);
  p = __builtin_fma(p, r, 1.0);
  return __builtin_ldexp(p, (int)n);
}
constexpr int kDMaxAll = 4096;  // grad_a keeps beta of every column in LDS, grad_b alpha of every row
typedef double mmd4 __attribute__((ext_vector_type(4)));

constexpr int kD64Fwd = 0, kD64GradA = 1, kD64GradB = 2;

__device__ __forceinline__ double d64_shift(double mx) { return mx == -INFINITY ? 0.0 : mx; }
__device__ __forceinline__ bool d64_usable(double shift) { return shift > 0.9 * kDFloor && shift < INFINITY; }

// kDT: tile edge, 64 (four waves, a wave's share 32 x 32) or 128 (eight waves, 32 x 64: every staged
// element - one exponential each - then feeds twice the products, and an item of 128 x 128 is one
// tile, so its maxima are taken once and its operands read once).  4 kDT threads.  tiles:
// (ceil(I / kDT), ceil(J / kDT)) per item; grid = B * tiles_i * tiles_j
template <int KIND, int kDT>
__device__ __forceinline__ void d64_log_mm_tile(double* __restrict__ smem64, int block, const double* __restrict__ a,
                                                const double* __restrict__ b, const double* __restrict__ out,
                                                const double* __restrict__ g, double* __restrict__ dst, int M,
                                                int K, int N, int tiles_i, int tiles_j) {
  constexpr bool FWD = KIND == kD64Fwd, GA = KIND == kD64GradA, GB = KIND == kD64GradB;
  const int I = GB ? K : M, J = FWD ? N : GA ? K : N, L = FWD ? K : GA ? N : M;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tile = block % (tiles_i * tiles_j), batch = block / (tiles_i * tiles_j);
  const int i0 = (tile / tiles_j) * kDT, j0 = (tile % tiles_j) * kDT;
  const double* ab = a + (long)batch * M * K;
  const double* bb = b + (long)batch * K * N;
  const double* ob = FWD ? nullptr : out + (long)batch * M * N;
  const double* gb = FWD ? nullptr : g + (long)batch * M * N;
  double* db = dst + (long)batch * I * J;

  constexpr int NT = 4 * kDT, kWaves = NT / 64;
  constexpr int kWI = 2, kWJ = kDT / 32;  // 16 x 16 accumulators per wave: rows, columns
  double* Ps = smem64;              // [kDT][kDP]: P[i][l]
  double* Qs = Ps + kDT * kDP;      // [kDT][kDP]: Q[l][j] as [j][l]
  double* al = Qs + kDT * kDP;      // alpha: the tile's rows m (forward, grad_a) or all M (grad_b)
  double* be = al + (GB ? M : kDT); // beta: the tile's columns n (forward, grad_b) or all N (grad_a)
  const int m_lo = GB ? 0 : i0, m_cnt = GB ? M : min(kDT, M - i0);
  const int n_lo = FWD ? j0 : GA ? 0 : j0, n_cnt = GA ? N : min(kDT, N - n_lo);

  // ---- maxima.  alpha: a wave per eight rows, lanes along k.  beta: 64 columns at a time, four
  // groups of 64 threads (one per wave) over k, combined through LDS (Ps is free yet).
  // (eight rows, resp. eight steps of k, are requested before the first is used: taken one at a
  // time, each waits out a full memory latency and the pre-pass costs a quarter of the kernel)
  for (int r0 = 8 * wave; r0 < m_cnt; r0 += 8 * kWaves) {
    double mx[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) mx[j] = -INFINITY;
    for (int k = lane; k < K; k += 64) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (r0 + j < m_cnt) mx[j] = fmax(mx[j], ab[(long)(m_lo + r0 + j) * K + k]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
#pragma unroll
      for (int s = 32; s >= 1; s >>= 1) mx[j] = fmax(mx[j], __shfl_xor(mx[j], s, 64));
      if (lane == 0 && r0 + j < m_cnt) al[r0 + j] = mx[j];
    }
  }
  for (int c0 = 0; c0 < n_cnt; c0 += 64) {
    const int c = c0 + lane;
    double mx = -INFINITY;
    if (c < n_cnt) {
#pragma unroll 8
      for (int k = wave; k < K; k += kWaves) mx = fmax(mx, bb[(long)k * N + n_lo + c]);
    }
    Ps[wave * 64 + lane] = mx;
    __syncthreads();
    if (wave == 0 && c < n_cnt) {
      double m = Ps[lane];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) m = fmax(m, Ps[64 * w + lane]);
      be[c] = m;
    }
    __syncthreads();
  }
  __syncthreads();

  // ---- staging.  A thread owns four neighbouring elements along the operand's contiguous
  // axis: (line = tid / 4, l = 4 (tid % 4) ..) where the contraction index is contiguous,
  // (l = tid / 16, line = 4 (tid % 16) ..) where the line index is.  raw_*: what memory
  // holds (the next chunk's, in flight during the products); put(): exponentials, LDS.
  constexpr bool P_L = !GB;  // P's contiguous axis is l (a[m][k] forward, g[m][n] grad_a); grad_b: i (a[m][k], i = k)
  constexpr bool Q_L = GA;   // Q's contiguous axis is l only in grad_a (b[k][n], l = n)
  constexpr int kLQ = kDT / 4;  // groups of four lines
  const int pl_line = P_L ? tid >> 2 : 4 * (tid % kLQ), pl_l = P_L ? 4 * (tid & 3) : tid / kLQ;
  const int ql_line = Q_L ? tid >> 2 : 4 * (tid % kLQ), ql_l = Q_L ? 4 * (tid & 3) : tid / kLQ;
  double rp[4], rp2[4], rq[4], rq2[4];
  auto load = [&](int l0) __attribute__((always_inline)) {
#pragma unroll
    for (int eh = 0; eh < 4; ++eh) {
      const int e = eh;
      {  // P[i][l]
        const int i = i0 + pl_line + (P_L ? 0 : e), l = l0 + pl_l + (P_L ? e : 0);
        const bool ok = i < I && l < L;
        long off = 0;
        if (FWD) off = (long)i * K + l;  // a[m = i][k = l]
        if (GA) off = (long)i * N + l;   // g, out [m = i][n = l]
        if (GB) off = (long)l * K + i;   // a[m = l][k = i]
        rp[eh] = ok ? (GA ? gb[off] : ab[off]) : 0.0;
        if (GA) rp2[eh] = ok ? ob[off] : 0.0;
      }
      {  // Q[l][j]
        const int j = j0 + ql_line + (Q_L ? 0 : e), l = l0 + ql_l + (Q_L ? e : 0);
        const bool ok = j < J && l < L;
        long off = 0;
        if (FWD) off = (long)l * N + j;  // b[k = l][n = j]
        if (GA) off = (long)j * N + l;   // b[k = j][n = l]
        if (GB) off = (long)l * N + j;   // g, out [m = l][n = j]
        rq[eh] = ok ? (GB ? gb[off] : bb[off]) : 0.0;
        if (GB) rq2[eh] = ok ? ob[off] : 0.0;
      }
    }
  };
  // H = g exp(alpha + beta - out); NaN where S = exp(out - alpha - beta) is not usable
  auto h_of = [&](double gv, double ov, double am, double bn) __attribute__((always_inline)) {
    const double sh = d64_shift(am) + d64_shift(bn), ls = ov - sh;  // ls = log S
    const bool ok = d64_usable(sh) && ls >= kDLogThr && ls < INFINITY;
    return ok ? gv * d64_exp(-ls) : __builtin_nan("");
  };
  auto put = [&](int l0) __attribute__((always_inline)) {
#pragma unroll
    for (int eh = 0; eh < 4; ++eh) {
      const int e = eh;
      {
        const int il = pl_line + (P_L ? 0 : e), ll = pl_l + (P_L ? e : 0);
        const int i = i0 + il, l = l0 + ll;
        // (computed for cells beyond the matrix too, then dropped: a select, not a branch)
        const int lc = min(l, L - 1);
        double v;
        if (FWD) v = d64_exp(rp[eh] - d64_shift(al[il]));
        if (GA) v = h_of(rp[eh], rp2[eh], al[il], be[lc]);
        if (GB) v = d64_exp(rp[eh] - d64_shift(al[lc]));
        Ps[il * kDP + ll] = (i < I && l < L) ? v : 0.0;
      }
      {
        const int jl = ql_line + (Q_L ? 0 : e), ll = ql_l + (Q_L ? e : 0);
        const int j = j0 + jl, l = l0 + ll;
        const int lc = min(l, L - 1);
        double v;
        if (FWD) v = d64_exp(rq[eh] - d64_shift(be[jl]));
        if (GA) v = d64_exp(rq[eh] - d64_shift(be[lc]));
        if (GB) v = h_of(rq[eh], rq2[eh], al[lc], be[jl]);
        Qs[jl * kDP + ll] = (j < J && l < L) ? v : 0.0;
      }
    }
  };

  // ---- products: wave (wi, wj) owns rows (kDT / 2) wi .., columns (kDT / 2) wj .. of the tile
  constexpr int kSI = 16 * kWI, kSJ = 16 * kWJ;  // a wave's rows and columns
  const int wi = wave >> 1, wj = wave & 1, l15 = lane & 15, zq = lane >> 4;
  mmd4 acc[kWI][kWJ];
#pragma unroll
  for (int x = 0; x < kWI; ++x)
#pragma unroll
    for (int y = 0; y < kWJ; ++y) acc[x][y] = mmd4{0.0, 0.0, 0.0, 0.0};
  load(0);
  for (int l0 = 0; l0 < L; l0 += kDC) {
    put(l0);
    __syncthreads();
    if (l0 + kDC < L) load(l0 + kDC);
#pragma unroll
    for (int ks = 0; ks < kDC / 4; ++ks) {
      double pa[kWI], qb[kWJ];
#pragma unroll
      for (int x = 0; x < kWI; ++x) pa[x] = Ps[(kSI * wi + 16 * x + l15) * kDP + 4 * ks + zq];
#pragma unroll
      for (int y = 0; y < kWJ; ++y) qb[y] = Qs[(kSJ * wj + 16 * y + l15) * kDP + 4 * ks + zq];
#pragma unroll
      for (int x = 0; x < kWI; ++x)
#pragma unroll
        for (int y = 0; y < kWJ; ++y) acc[x][y] = __builtin_amdgcn_mfma_f64_16x16x4f64(pa[x], qb[y], acc[x][y], 0, 0, 0);
    }
    __syncthreads();
  }

  // ---- results: accumulator element r of tile (x, y) is row kSI wi + 16 x + 4 r + zq, column
  // kSJ wj + 16 y + l15
#pragma unroll
  for (int x = 0; x < kWI; ++x)
#pragma unroll
    for (int y = 0; y < kWJ; ++y)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int il = kSI * wi + 16 * x + 4 * r + zq, jl = kSJ * wj + 16 * y + l15;
        const int i = i0 + il, j = j0 + jl;
        if (i >= I || j >= J) continue;
        const double v = acc[x][y][r];
        double res;
        if (FWD) {
          const double sh = d64_shift(al[il]) + d64_shift(be[jl]);
          if (d64_usable(sh) && v >= kDThr && v < INFINITY) {
            res = log(v) + sh;
          } else {  // the reference's two passes (matmul_cuda_kernel.cu:27-41)
            const double* arow = ab + (long)i * K;
            const double* bcol = bb + j;
            double mx = kDFloor;
            for (int k = 0; k < K; ++k) mx = fmax(mx, arow[k] + bcol[(long)k * N]);
            double s = 0.0;
            for (int k = 0; k < K; ++k) s += exp(arow[k] + bcol[(long)k * N] - mx);
            res = log(s) + mx;
          }
        } else if (GA) {  // i = m, j = k
          const double av = ab[(long)i * K + j];
          res = d64_exp(av - d64_shift(al[il])) * v;
          if (!(fabs(res) <= DBL_MAX)) {  // matmul_cuda_kernel.cu:159-184
            double s = 0.0;
            for (int n = 0; n < N; ++n)
              s = __builtin_fma(exp(av + bb[(long)j * N + n] - ob[(long)i * N + n]), gb[(long)i * N + n], s);
            res = s;
          }
        } else {  // i = k, j = n
          const double bv = bb[(long)i * N + j];
          res = d64_exp(bv - d64_shift(be[jl])) * v;
          if (!(fabs(res) <= DBL_MAX)) {  // matmul_cuda_kernel.cu:190-217
            double s = 0.0;
            for (int m = 0; m < M; ++m)
              s = __builtin_fma(exp(ab[(long)m * K + i] + bv - ob[(long)m * N + j]), gb[(long)m * N + j], s);
            res = s;
          }
        }
        db[(long)i * J + j] = res;
      }
}

template <int KIND, int kDT>
__global__ __launch_bounds__(4 * kDT, 4) void k64_log_mm(const double* __restrict__ a, const double* __restrict__ b,
                                                         const double* __restrict__ out,
                                                         const double* __restrict__ g, double* __restrict__ dst,
                                                         int M, int K, int N, int tiles_i, int tiles_j) {
  extern __shared__ __attribute__((aligned(16))) double smem64[];
  d64_log_mm_tile<KIND, kDT>(smem64, blockIdx.x, a, b, out, g, dst, M, K, N, tiles_i, tiles_j);
}

// Both gradients of items that are one tile each, in one launch.  Workgroups come in groups of
// 16: the first eight take grad_a of eight consecutive items, the next eight grad_b of the same
// items (workgroup w runs on XCD w mod 8, so an item's second reader finds a, b, out and g in that
// XCD's L2).
template <int kDT>
__global__ __launch_bounds__(4 * kDT, 4) void k64_log_mm_both(const double* __restrict__ a,
                                                              const double* __restrict__ b,
                                                              const double* __restrict__ out,
                                                              const double* __restrict__ g,
                                                              double* __restrict__ grad_a,
                                                              double* __restrict__ grad_b, int B, int M, int K,
                                                              int N) {
  extern __shared__ __attribute__((aligned(16))) double smem64[];
  const int w = blockIdx.x, item = (w >> 4) * 8 + (w & 7);
  if (item >= B) return;
  if (((w >> 3) & 1) == 0) d64_log_mm_tile<kD64GradA, kDT>(smem64, item, a, b, out, g, grad_a, M, K, N, 1, 1);
  else d64_log_mm_tile<kD64GradB, kDT>(smem64, item, a, b, out, g, grad_b, M, K, N, 1, 1);
}

inline size_t d64_mm_lds(int kind, int tile, int M, int N) {
  return sizeof(double) * (2 * tile * kDP + (kind == kD64GradB ? M : tile) + (kind == kD64GradA ? N : tile));
}

}  // namespace GENBMM_NS
