// logbmm for small matrices (M, K, N <= 64): one workgroup per batch item, the
// whole item in LDS, one launch for the forward and one for both gradients.
// At these sizes the problem is launch- and HBM-bound (a 32^3 item is 12 KB of
// operands and 0.2 M products), so the kernels read every operand exactly once
// and write every result exactly once, in contiguous runs.
//
// Same factored form as the large kernels: alpha[m] = max_k a, beta[n] = max_k b
// are taken inside the workgroup, EA = exp(a - alpha), EB = exp(b - beta),
// S = EA * EB, out = log S + alpha + beta, H = g * exp(alpha + beta - out),
// grad_a = EA .* (H * EB^T), grad_b = EB .* (EA^T * H).  A cell (forward) or an
// item (backward) for which the factoring is not exact to fp32 - S < 2^-40, a
// shift at the reference's -1e9 floor, anything non-finite - is recomputed inside
// the same kernel from global memory with the reference's own two-pass form.
#pragma once

#include "common.h"
#include "logbmm_ws.h"

namespace GENBMM_NS {

constexpr float kItemGuardBits = 40.f;

// log-sum-exp of a[m,:] + b[:,n] the way the reference's kernel does it
// (matmul_cuda_kernel.cu:27-41): running maximum from -1e9, then the sum.
__device__ __forceinline__ float item_exact_out(const elem_t* __restrict__ arow,
                                                const elem_t* __restrict__ bcol, int K, int N) {
  float mx = kFloor;
  for (int k = 0; k < K; ++k) mx = fmaxf(mx, (float)arow[k] + (float)bcol[(long)k * N]);
  const float nm = -mx * kLog2e;
  float s = 0.f;
  for (int k = 0; k < K; ++k)
    s += fast_exp2(__builtin_fmaf((float)arow[k] + (float)bcol[(long)k * N], kLog2e, nm));
  return logf(s) + mx;
}

// (row, column) of elements tid, tid + nt, tid + 2 nt, ... of a row-major array
// with C columns, without a division per element.
struct RowMajorWalk {
  int r, c, dr, dc, C;
  __device__ __forceinline__ RowMajorWalk(int tid, int nt, int cols) : C(cols) {
    r = tid / C;
    c = tid - r * C;
    dr = nt / C;
    dc = nt - dr * C;
  }
  __device__ __forceinline__ void next() {
    r += dr;
    c += dc;
    if (c >= C) {
      c -= C;
      ++r;
    }
  }
};

// exp(x - shift), with the all -inf row / column (shift = -inf) giving zeros
__device__ __forceinline__ float item_exp(float x, float shift) {
  return fast_exp2((x - (shift == -INFINITY ? 0.f : shift)) * kLog2e);
}

// TB x TB outputs per thread on a G x G thread grid.  Used with G = 16: TB = 2
// covers items up to 32 x 32, TB = 4 up to 64 x 64.  (One wave per item, G = 8 and
// TB = 4, measured slower at 8192 items of 32^3: the chain of dependent phases of
// an item gets longer than the extra items in flight make up for.)
// FULL: M = K = N = G * TB, known to the compiler - the index arithmetic that is most of
// the general kernel's instructions (it is issue-bound, not memory-bound) folds away.
template <int G, int TB, bool FULL = false>
__global__ __launch_bounds__(G * G, TB == 2 ? 8 : 1) void k_log_item_fwd(const elem_t* __restrict__ a,
                                                      const elem_t* __restrict__ b,
                                                      elem_t* __restrict__ out,
                                                      float* __restrict__ stats,
                                                      int* __restrict__ hdr, int M_, int K_,
                                                      int N_) {
  constexpr int NT = G * G, S = G * TB, LD = S + 1;
  const int M = FULL ? S : M_, K = FULL ? S : K_, N = FULL ? S : N_;
  static_assert(2 * S <= NT, "row and column scans use 2*S threads");
  if (hdr && blockIdx.x == 0 && threadIdx.x == 0) hdr[0] = kWsNone;  // no per-tile flags in this workspace
  __shared__ float At[S * LD];  // [k][m]: a, then EA; finally the output tile [m][n]
  __shared__ float Bs[S * LD];  // [k][n]: b, then EB
  __shared__ float al[S], be[S];
  const int tid = threadIdx.x, batch = blockIdx.x;
  const elem_t* ab = a + (long)batch * M * K;
  const elem_t* bb = b + (long)batch * K * N;
  // All reads of the item are issued before the first one is waited for (a thread owns
  // elements tid, tid + NT, ... of each operand): one trip to memory, not one per element.
  constexpr int PER = TB * TB;  // S * S / NT
  float ra[PER], rb[PER];
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int e = tid + u * NT;
    ra[u] = e < M * K ? ab[e] : 0.f;
    rb[u] = e < K * N ? bb[e] : 0.f;
  }
  {
    RowMajorWalk w(tid, NT, K);
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      if (w.r < M) At[w.c * LD + w.r] = ra[u];
      w.next();
    }
  }
  {
    RowMajorWalk w(tid, NT, N);
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      if (w.r < K) Bs[w.r * LD + w.c] = rb[u];
      w.next();
    }
  }
  __syncthreads();
  // row / column maxima: one thread per row, one per column (LDS atomics on the
  // shared maximum while loading measured slower: 32 lanes on one address)
  if (tid < M) {
    float mx = -INFINITY;
    for (int k = 0; k < K; ++k) mx = fmaxf(mx, At[k * LD + tid]);
    al[tid] = mx;
  } else if (tid >= S && tid - S < N) {
    float mx = -INFINITY;
    for (int k = 0; k < K; ++k) mx = fmaxf(mx, Bs[k * LD + tid - S]);
    be[tid - S] = mx;
  }
  __syncthreads();
  for (RowMajorWalk w(tid, NT, K); w.r < M; w.next()) {
    const int m = w.r, k = w.c;
    At[k * LD + m] = item_exp(At[k * LD + m], al[m]);
  }
  for (RowMajorWalk w(tid, NT, N); w.r < K; w.next()) {
    const int k = w.r, n = w.c, e = w.r * N + w.c;
    Bs[k * LD + n] = item_exp(Bs[k * LD + n], be[n]);
  }
  if (stats) {
    float* st = stats + (long)batch * (M + N);
    if (tid < M) st[tid] = al[tid];
    else if (tid >= S && tid - S < N) st[M + tid - S] = be[tid - S];
  }
  __syncthreads();

  const int ty = tid / G, tx = tid % G;
  float acc[TB][TB];
#pragma unroll
  for (int i = 0; i < TB; ++i)
#pragma unroll
    for (int j = 0; j < TB; ++j) acc[i][j] = 0.f;
#pragma unroll 4
  for (int k = 0; k < K; ++k) {
    float av[TB], bv[TB];
#pragma unroll
    for (int i = 0; i < TB; ++i) av[i] = At[k * LD + ty * TB + i];
#pragma unroll
    for (int j = 0; j < TB; ++j) bv[j] = Bs[k * LD + tx * TB + j];
#pragma unroll
    for (int i = 0; i < TB; ++i)
#pragma unroll
      for (int j = 0; j < TB; ++j) acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
  }
  __syncthreads();  // At becomes the output tile
  const float thr = fast_exp2(-kItemGuardBits);
#pragma unroll
  for (int i = 0; i < TB; ++i)
#pragma unroll
    for (int j = 0; j < TB; ++j) {
      const int m = ty * TB + i, n = tx * TB + j;
      if (m < M && n < N) {
        const float shift = al[m] + be[n], s = acc[i][j];
        const bool ok = (s >= thr) && (s < INFINITY) && (shift >= kFloor) && (shift < INFINITY);
        At[m * LD + n] = ok ? __builtin_fmaf(fast_log2(s), kLn2, shift)
                            : item_exact_out(ab + (long)m * K, bb + n, K, N);
      }
    }
  __syncthreads();
  elem_t* ob = out + (long)batch * M * N;
  for (RowMajorWalk w(tid, NT, N); w.r < M; w.next()) {
    const int m = w.r, n = w.c, e = w.r * N + w.c;
    ob[e] = to_elem<elem_t>(At[m * LD + n]);
  }
}

template <int G, int TB, bool FULL = false>
__global__ __launch_bounds__(G * G, TB == 2 ? 6 : 1) void k_log_item_bwd(const elem_t* __restrict__ a,
                                                      const elem_t* __restrict__ b,
                                                      const elem_t* __restrict__ outp,
                                                      const elem_t* __restrict__ g,
                                                      elem_t* __restrict__ grad_a,
                                                      elem_t* __restrict__ grad_b, int M_, int K_,
                                                      int N_) {
  constexpr int NT = G * G, S = G * TB, LD = S + 1;
  const int M = FULL ? S : M_, K = FULL ? S : K_, N = FULL ? S : N_;
  static_assert(2 * S <= NT, "row and column scans use 2*S threads");
  __shared__ float Ea[S * LD];  // [m][k]: a, EA, finally grad_a
  __shared__ float Eb[S * LD];  // [k][n]: b, EB, finally grad_b
  __shared__ float Hs[S * LD];  // [m][n]: H
  __shared__ float al[S], be[S];
  const int tid = threadIdx.x, batch = blockIdx.x;
  const elem_t* ab = a + (long)batch * M * K;
  const elem_t* bb = b + (long)batch * K * N;
  const elem_t* ob = outp + (long)batch * M * N;
  const elem_t* gb = g + (long)batch * M * N;
  elem_t* gab = grad_a ? grad_a + (long)batch * M * K : nullptr;
  elem_t* gbb = grad_b ? grad_b + (long)batch * K * N : nullptr;
  // all reads of the item in flight together (see the forward)
  constexpr int PER = TB * TB;
  float ra[PER], rb[PER], ro[PER], rg[PER];
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int e = tid + u * NT;
    ra[u] = e < M * K ? ab[e] : 0.f;
    rb[u] = e < K * N ? bb[e] : 0.f;
    ro[u] = e < M * N ? ob[e] : 0.f;
    rg[u] = e < M * N ? gb[e] : 0.f;
  }
  {
    RowMajorWalk w(tid, NT, K);
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      if (w.r < M) Ea[w.r * LD + w.c] = ra[u];
      w.next();
    }
  }
  {
    RowMajorWalk w(tid, NT, N);
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      if (w.r < K) Eb[w.r * LD + w.c] = rb[u];
      w.next();
    }
  }
  __syncthreads();
  if (tid < M) {
    float mx = -INFINITY;
    for (int k = 0; k < K; ++k) mx = fmaxf(mx, Ea[tid * LD + k]);
    al[tid] = mx;
  } else if (tid >= S && tid - S < N) {
    float mx = -INFINITY;
    for (int k = 0; k < K; ++k) mx = fmaxf(mx, Eb[k * LD + tid - S]);
    be[tid - S] = mx;
  }
  __syncthreads();
  const float lim = kItemGuardBits * kLn2 + 1e-3f;
  int bad = 0;
  for (RowMajorWalk w(tid, NT, K); w.r < M; w.next()) {
    const int m = w.r, k = w.c, e = w.r * K + w.c;
    Ea[m * LD + k] = item_exp(Ea[m * LD + k], al[m]);
  }
  for (RowMajorWalk w(tid, NT, N); w.r < K; w.next()) {
    const int k = w.r, n = w.c, e = w.r * N + w.c;
    Eb[k * LD + n] = item_exp(Eb[k * LD + n], be[n]);
  }
  {
    RowMajorWalk w(tid, NT, N);
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      if (w.r < M) {
        const int m = w.r, n = w.c;
        const float ex = al[m] + be[n] - ro[u];
        if (!(ex <= lim) || !(ex > -INFINITY)) bad = 1;  // S < 2^-40, NaN or infinities: not exact
        Hs[m * LD + n] = rg[u] * fast_exp2(ex * kLog2e);
      }
      w.next();
    }
  }
  bad = __syncthreads_or(bad);
  if (bad) {
    // the reference's form for the whole item (matmul_cuda_kernel.cu:159-184):
    // exp(a + b - out) * g summed over n (grad_a) / m (grad_b), from global memory
    if (gab)
      for (int e = tid; e < M * K; e += NT) {
        const int m = e / K, k = e - m * K;
        const float av = ab[e];
        float s = 0.f;
        for (int n = 0; n < N; ++n)
          s = __builtin_fmaf(fast_exp(av + (float)bb[(long)k * N + n] - (float)ob[(long)m * N + n]), (float)gb[(long)m * N + n], s);
        gab[e] = to_elem<elem_t>(s);
      }
    if (gbb)
      for (int e = tid; e < K * N; e += NT) {
        const int k = e / N, n = e - k * N;
        const float bv = bb[e];
        float s = 0.f;
        for (int m = 0; m < M; ++m)
          s = __builtin_fmaf(fast_exp((float)ab[(long)m * K + k] + bv - (float)ob[(long)m * N + n]), (float)gb[(long)m * N + n], s);
        gbb[e] = to_elem<elem_t>(s);
      }
    return;
  }

  const int ty = tid / G, tx = tid % G;
  float ga[TB][TB], gw[TB][TB];
#pragma unroll
  for (int i = 0; i < TB; ++i)
#pragma unroll
    for (int j = 0; j < TB; ++j) ga[i][j] = gw[i][j] = 0.f;
  if (gab) {  // rows m = ty*TB+i, columns k = tx*TB+j, sum over n
#pragma unroll 4
    for (int n = 0; n < N; ++n) {
      float hv[TB], ev[TB];
#pragma unroll
      for (int i = 0; i < TB; ++i) hv[i] = Hs[(ty * TB + i) * LD + n];
#pragma unroll
      for (int j = 0; j < TB; ++j) ev[j] = Eb[(tx * TB + j) * LD + n];
#pragma unroll
      for (int i = 0; i < TB; ++i)
#pragma unroll
        for (int j = 0; j < TB; ++j) ga[i][j] = __builtin_fmaf(hv[i], ev[j], ga[i][j]);
    }
  }
  if (gbb) {  // rows k = ty*TB+i, columns n = tx*TB+j, sum over m
#pragma unroll 4
    for (int m = 0; m < M; ++m) {
      float ev[TB], hv[TB];
#pragma unroll
      for (int i = 0; i < TB; ++i) ev[i] = Ea[m * LD + ty * TB + i];
#pragma unroll
      for (int j = 0; j < TB; ++j) hv[j] = Hs[m * LD + tx * TB + j];
#pragma unroll
      for (int i = 0; i < TB; ++i)
#pragma unroll
        for (int j = 0; j < TB; ++j) gw[i][j] = __builtin_fmaf(ev[i], hv[j], gw[i][j]);
    }
  }
  __syncthreads();  // all sums taken: scale in place, each thread its own cells
#pragma unroll
  for (int i = 0; i < TB; ++i)
#pragma unroll
    for (int j = 0; j < TB; ++j) {
      const int r = ty * TB + i, c = tx * TB + j;
      Ea[r * LD + c] *= ga[i][j];
      Eb[r * LD + c] *= gw[i][j];
    }
  __syncthreads();
  if (gab)
    for (RowMajorWalk w(tid, NT, K); w.r < M; w.next()) gab[w.r * K + w.c] = to_elem<elem_t>(Ea[w.r * LD + w.c]);
  if (gbb)
    for (RowMajorWalk w(tid, NT, N); w.r < K; w.next()) gbb[w.r * N + w.c] = to_elem<elem_t>(Eb[w.r * LD + w.c]);
}

}  // namespace GENBMM_NS
