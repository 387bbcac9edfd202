// logbmm second order (gfx950): gradients with respect to (a, b, g) of
// <u_a, grad_a> + <u_b, grad_b>, where (grad_a, grad_b) are the first-order gradients for the
// incoming gradient g.  Replaces _genbmm.backbackward (matmul_cuda.cpp:94-109,
// matmul_cuda_kernel.cu:547-622, kernels :220-331).
//
// With p = exp(a[m,k] + b[k,n] - out[m,n]), w = u_a[m,k] + u_b[k,n] (a missing u counts as 0):
//   t[m,n]      = sum_k p * w                        (gradient w.r.t. g)
//   grad_a[m,k] = sum_n g[m,n] * p * (w - t[m,n])
//   grad_b[k,n] = sum_m g[m,n] * p * (w - t[m,n])
// With u_b = 0 these are the reference's three quartic kernels (inner = sum_k2 (delta*s -
// s*s2)*u[k2] = s*(u[k] - t)) in O(M K N).
//
// Two implementations.
//  * Exact, on the vector ALU: three passes (t, grad_a, grad_b), one exponential per (m,k,n)
//    in each.  Any shape; the whole computation for small problems, and the recompute of
//    batch items that the factored form cannot take.
//  * Factored, on the fp32 matrix cores (needs the caller's workspace): with the row maxima
//    alpha of a and column maxima beta of b, EA = exp(a - alpha), EB = exp(b - beta),
//    R = exp(alpha + beta - out), H = g R, X = EA u_a, Y = EB u_b:
//      t      = R (X EB + EA Y)
//      grad_a = X (H EB^T) + EA (H Y^T - (H t) EB^T)
//      grad_b = Y (EA^T H) + EB (X^T H - EA^T (H t))
//    eight products (five when u_b is absent) of batched GEMM shape.  The operands are laid out
//    once, zero-padded to multiples of 128 in every extent, by three elementwise passes; one
//    GEMM kernel (128 x 128 tiles of v_mfma_f32_32x32x2_f32, 16-deep slabs through two LDS
//    buffers) then runs without any edge handling in its loop, sums up to two products into one
//    accumulator and applies the epilogue of its role.  A batch item with a cell whose
//    alpha + beta - out is beyond 40 ln 2 or not finite (a factor could underflow against a
//    term that matters) is flagged by the pass that forms H and redone by the exact kernels,
//    which run behind the factored ones on the flagged items only.
#include <algorithm>
#include <type_traits>

#include "logbmm_mfma.h"

namespace GENBMM_NS {
namespace {

// ------------------------------------------------------------------ exact passes
// tt: t per output cell as float (grad_g itself for float tensors; a buffer of the workspace for
// the half types, whose grad_g holds t rounded).  only: NULL, or one word per batch item - items
// whose word is 0 are skipped.
struct BB {
  const elem_t* a; const elem_t* b; const elem_t* out; const elem_t* g;
  const elem_t* ua; const elem_t* ub;
  elem_t* ga; elem_t* gb; elem_t* gg;
  float* tt;
  const int* only;
  int M, K, N;
  int B;
};

// The blocks of a pass.  A block is `per_block` consecutive units (cells or rows) starting at `base`
// and ending before `limit`; f(base, limit) works on one.  Without `only`: one block per workgroup
// over all units (numbered so that an item's workgroups share an XCD).  With it - the pass over
// flagged items, which usually finds none - a small grid reads the flags 64 at a time; its workgroups
// form groups of one item's blocks (or one group that strides, for items of more blocks than the
// grid), and the flagged items go to the groups in turn: tens of thousands of workgroups that look
// up a flag and exit cost 60 us a launch, this costs 2.
constexpr int kBBOnlyGrid = 2048;
template <bool ONLY, class F>
__device__ __forceinline__ void bb_blocks(const BB& p, long total, long per_item, int per_block, F&& f) {
  if constexpr (!ONLY) {
    f((long)xcd_renumber(blockIdx.x, gridDim.x) * per_block, total);
    return;
  }
  const int lane = threadIdx.x & 63;
  const long bpi = (per_item + per_block - 1) / per_block;  // blocks per item
  const bool fits = bpi <= (long)gridDim.x;
  const long groups = fits ? (long)gridDim.x / bpi : 1;
  const long grp = fits ? (long)blockIdx.x / bpi : 0;
  if (grp >= groups) return;
  const long first = fits ? (long)blockIdx.x - grp * bpi : (long)blockIdx.x;
  const long stride = fits ? bpi : (long)gridDim.x;
  long seen = 0;
  for (int b0 = 0; b0 < p.B; b0 += 64) {
    unsigned long long live = __ballot(b0 + lane < p.B && p.only[b0 + lane] != 0);
    while (live) {
      const long batch = b0 + __builtin_ctzll(live);
      live &= live - 1;
      if (seen++ % groups != grp) continue;
      for (long u = first * per_block; u < per_item; u += stride * per_block)
        f(batch * per_item + u, (batch + 1) * per_item);
    }
  }
}
inline dim3 bb_grid(const BB& p, long nblocks) {
  return dim3((unsigned)(p.only ? std::min<long>(nblocks, kBBOnlyGrid) : nblocks));
}

template <bool ONLY>
__global__ __launch_bounds__(256) void k_log_bwdbwd_t(const BB p, long total) {
  bb_blocks<ONLY>(p, total, (long)p.M * p.N, 256, [&](long base, long limit) __attribute__((always_inline)) {
  const long e = base + threadIdx.x;
  if (e >= limit) return;
  const int n = (int)(e % p.N);
  const long bm = e / p.N;  // batch*M + m
  const long batch = bm / p.M;
  if (p.only && !p.only[batch]) return;
  const elem_t* arow = p.a + bm * p.K;
  const elem_t* uarow = p.ua ? p.ua + bm * p.K : nullptr;
  const elem_t* bcol = p.b + batch * p.K * p.N + n;
  const elem_t* ubcol = p.ub ? p.ub + batch * p.K * p.N + n : nullptr;
  const float o = p.out[e];
  float t = 0.f;
  for (int k = 0; k < p.K; ++k) {
    const float pr = fast_exp((float)arow[k] + (float)bcol[(long)k * p.N] - o);
    const float w = (uarow ? (float)uarow[k] : 0.f) + (ubcol ? (float)ubcol[(long)k * p.N] : 0.f);
    t = __builtin_fmaf(pr, w, t);
  }
  p.tt[e] = t;
  if constexpr (!kElemF32) p.gg[e] = to_elem<elem_t>(t);
  });
}

// grad_a: a wave per row (batch, m), its lanes along n - the one axis on which b, u_b, out, g and
// t are all contiguous (with a lane per cell (m, k) the reads of b run down a column, one cache
// line per lane).  The row's out, g and t stay in registers for N <= 256; per k the lanes'
// partial sums are added across the wave and 64 finished cells are written at once.
constexpr int kBBChunks = 4;  // n chunks of 64 a lane keeps in registers
template <bool ONLY>
__global__ __launch_bounds__(256) void k_log_bwdbwd_a(const BB p, long rows) {
  bb_blocks<ONLY>(p, rows, (long)p.M, 4, [&](long base, long limit) __attribute__((always_inline)) {
  const int lane = threadIdx.x & 63;
  const long bm = base + (threadIdx.x >> 6);
  if (bm >= limit) return;
  const long batch = bm / p.M;
  if (p.only && !p.only[batch]) return;
  const int K = p.K, N = p.N;
  const elem_t* arow = p.a + bm * K;
  const elem_t* uarow = p.ua ? p.ua + bm * K : nullptr;
  const elem_t* bmat = p.b + batch * K * N;
  const elem_t* ubmat = p.ub ? p.ub + batch * K * N : nullptr;
  const elem_t* orow = p.out + bm * N;
  const elem_t* grow = p.g + bm * N;
  const float* trow = p.tt + bm * N;
  const bool cached = N <= 64 * kBBChunks;
  float oc[kBBChunks], gc[kBBChunks], tc[kBBChunks];
#pragma unroll
  for (int j = 0; j < kBBChunks; ++j) {
    const int n = lane + 64 * j;
    const bool in = cached && n < N;
    oc[j] = in ? (float)orow[n] : 0.f;
    gc[j] = in ? (float)grow[n] : 0.f;
    tc[j] = in ? trow[n] : 0.f;
  }
  float mine = 0.f;  // the finished cell k with k % 64 == lane
  for (int k = 0; k < K; ++k) {
    const float av = arow[k], uav = uarow ? (float)uarow[k] : 0.f;
    const elem_t* brow = bmat + (long)k * N;
    const elem_t* ubrow = ubmat ? ubmat + (long)k * N : nullptr;
    float acc = 0.f;
    if (cached) {
#pragma unroll
      for (int j = 0; j < kBBChunks; ++j) {
        const int n = lane + 64 * j;
        if (n < N) {
          const float pr = fast_exp(av + (float)brow[n] - oc[j]);
          const float w = uav + (ubrow ? (float)ubrow[n] : 0.f) - tc[j];
          acc = __builtin_fmaf(gc[j] * pr, w, acc);
        }
      }
    } else {
      for (int n = lane; n < N; n += 64) {
        const float pr = fast_exp(av + (float)brow[n] - (float)orow[n]);
        const float w = uav + (ubrow ? (float)ubrow[n] : 0.f) - trow[n];
        acc = __builtin_fmaf((float)grow[n] * pr, w, acc);
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if ((k & 63) == lane) mine = acc;
    if ((k & 63) == 63 || k == K - 1) {
      const int k0 = k & ~63;
      if (k0 + lane <= k) p.ga[bm * K + k0 + lane] = to_elem<elem_t>(mine);
    }
  }
  });
}

template <bool ONLY>
__global__ __launch_bounds__(256) void k_log_bwdbwd_b(const BB p, long total) {
  bb_blocks<ONLY>(p, total, (long)p.K * p.N, 256, [&](long base, long limit) __attribute__((always_inline)) {
  const long e = base + threadIdx.x;
  if (e >= limit) return;
  const int n = (int)(e % p.N);
  const long bk = e / p.N;  // batch*K + k
  const long batch = bk / p.K;
  if (p.only && !p.only[batch]) return;
  const int k = (int)(bk - batch * p.K);
  const float bv = p.b[e];
  const float ubv = p.ub ? (float)p.ub[e] : 0.f;
  const elem_t* acol = p.a + batch * p.M * p.K + k;
  const elem_t* uacol = p.ua ? p.ua + batch * p.M * p.K + k : nullptr;
  const elem_t* ocol = p.out + batch * p.M * p.N + n;
  const elem_t* gcol = p.g + batch * p.M * p.N + n;
  const float* tcol = p.tt + batch * p.M * p.N + n;
  float acc = 0.f;
  for (int m = 0; m < p.M; ++m) {
    const long mn = (long)m * p.N;
    const float pr = fast_exp((float)acol[(long)m * p.K] + bv - (float)ocol[mn]);
    const float w = (uacol ? (float)uacol[(long)m * p.K] : 0.f) + ubv - tcol[mn];
    acc = __builtin_fmaf((float)gcol[mn] * pr, w, acc);
  }
  p.gb[e] = to_elem<elem_t>(acc);
  });
}

int launch_exact(const BB& p, int B, hipStream_t s) {
  auto blocks = [&](long total) { return bb_grid(p, (total + 255) / 256); };
  const long tmn = (long)B * p.M * p.N, tmk = (long)B * p.M * p.K, tkn = (long)B * p.K * p.N;
  if (tmn > 0) {
    hipLaunchKernelGGL(p.only ? k_log_bwdbwd_t<true> : k_log_bwdbwd_t<false>, blocks(tmn), dim3(256), 0, s, p, tmn);
    if (int e = launch_status()) return e;
  }
  if (tmk > 0) {
    const long rows = (long)B * p.M;  // four rows per workgroup
    hipLaunchKernelGGL(p.only ? k_log_bwdbwd_a<true> : k_log_bwdbwd_a<false>, bb_grid(p, (rows + 3) / 4), dim3(256), 0, s,
                       p, rows);
    if (int e = launch_status()) return e;
  }
  if (tkn > 0) {
    hipLaunchKernelGGL(p.only ? k_log_bwdbwd_b<true> : k_log_bwdbwd_b<false>, blocks(tkn), dim3(256), 0, s, p, tkn);
    if (int e = launch_status()) return e;
  }
  return GENBMM_OK;
}

// ------------------------------------------------------------------ factored form
constexpr int kBBPad = 128;  // every extent of the workspace's arrays is a multiple of this
inline int bb_pad(int x) { return (x + kBBPad - 1) / kBBPad * kBBPad; }
// The factored form pays from here on (padding to 128 at most doubles an extent of 64).
inline bool bb_factored_ok(int B, int M, int K, int N) {
  return min(M, min(K, N)) >= 64 && (int64_t)B * M * K * N >= ((int64_t)1 << 21);
}

struct BBWs {
  float* t_exact;  // (B, M, N): t for the exact passes (and unrounded for the half types)
  float* alpha;    // (B, Mp)
  float* beta;     // (B, Np)
  int* flags;      // (B): items to redo exactly
  float *ea, *x;   // (B, Mp, Kp): exp(a - alpha), ea * u_a
  float *eb, *y;   // (B, Kp, Np)
  float *r, *h, *nht;  // (B, Mp, Np): exp(alpha + beta - out), g r, -h t
  float *ga0;      // (B, Mp, Kp): H EB^T
  float *gb0;      // (B, Kp, Np): EA^T H
};
inline size_t bb_ws_floats(int B, int M, int K, int N, BBWs* w, float* base) {
  size_t off = 0;
  auto take = [&](size_t n) {
    float* p = base ? base + off : nullptr;
    off += (n + 3) & ~(size_t)3;
    return p;
  };
  BBWs t{};
  t.t_exact = take((size_t)B * M * N);
  if (bb_factored_ok(B, M, K, N)) {
    const size_t Mp = bb_pad(M), Kp = bb_pad(K), Np = bb_pad(N);
    t.alpha = take(B * Mp);
    t.beta = take(B * Np);
    t.flags = reinterpret_cast<int*>(take(B));
    t.ea = take(B * Mp * Kp); t.x = take(B * Mp * Kp);
    t.eb = take(B * Kp * Np); t.y = take(B * Kp * Np);
    t.r = take(B * Mp * Np); t.h = take(B * Mp * Np); t.nht = take(B * Mp * Np);
    t.ga0 = take(B * Mp * Kp);
    t.gb0 = take(B * Kp * Np);
  }
  if (w) *w = t;
  return off;
}

// The three passes move four cells per lane and instruction (the padded extents are multiples of
// 128; rows of the caller's tensors start at any element, which the loads take).
__device__ __forceinline__ float4 exp4_st(float4 v, float m) {
  return make_float4(exp_st(v.x - m), exp_st(v.y - m), exp_st(v.z - m), exp_st(v.w - m));
}
__device__ __forceinline__ float4 mul4(float4 a, float4 b) { return make_float4(a.x * b.x, a.y * b.y, a.z * b.z, a.w * b.w); }
__device__ __forceinline__ float max4(float m, float4 v) { return fmaxf(fmaxf(m, fmaxf(v.x, v.y)), fmaxf(v.z, v.w)); }

// alpha, EA, X: a wave per padded row (b, mp) - half a wave where a row is 128 cells, 32 lanes' worth;
// rows and columns of the padding hold zeros.
__global__ __launch_bounds__(256) void k_bb_prep_a(const elem_t* __restrict__ a, const elem_t* __restrict__ ua,
                                                   float* __restrict__ alpha, float* __restrict__ ea,
                                                   float* __restrict__ x, int* __restrict__ flags, int M, int K,
                                                   int Mp, int Kp, long rows) {
  const int lpr = Kp == 128 ? 32 : 64;  // lanes per row
  const int lane = threadIdx.x & (lpr - 1);
  const long row = ((long)blockIdx.x * 256 + threadIdx.x) / lpr;
  if (row >= rows) return;
  const long batch = row / Mp;
  const int m = (int)(row - batch * Mp);
  if (row < (rows / Mp) && lane == 0) flags[row] = 0;  // (rows / Mp = B words, cleared by the first B rows)
  float* er = ea + row * Kp;
  float* xr = x + row * Kp;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  const int step = lpr * 4;
  if (m >= M) {
    for (int k = lane * 4; k < Kp; k += step) { st4(er + k, zero); st4(xr + k, zero); }
    if (lane == 0) alpha[row] = 0.f;
    return;
  }
  const elem_t* ar = a + (batch * M + m) * K;
  const elem_t* ur = ua ? ua + (batch * M + m) * K : nullptr;
  float mx = -INFINITY;
  for (int k = lane * 4; k < K; k += step) mx = max4(mx, ld4m(ar + k, K - k, -INFINITY));
  // (the exchange stays within the row's own lanes, all of which are here)
#pragma unroll
  for (int off = 32; off > 0; off >>= 1)
    if (off < lpr) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
  if (lane == 0) alpha[row] = mx;
  for (int k = lane * 4; k < Kp; k += step) {
    // (the fill -inf gives exp = 0 in the padding; a row of -inf has mx = -inf and NaN here, and is
    //  flagged by the pass that forms H)
    const float4 e = k < K ? exp4_st(ld4m(ar + k, K - k, -INFINITY), mx) : zero;
    st4(er + k, e);
    st4(xr + k, (ur && k < K) ? mul4(e, ld4m(ur + k, K - k, 0.f)) : zero);
  }
}

// beta, EB, Y: a workgroup per (batch item, 64 columns): 16 lanes x 4 columns across, the 16 lane
// groups of the four waves split the rows of b.
__global__ __launch_bounds__(256) void k_bb_prep_b(const elem_t* __restrict__ b, const elem_t* __restrict__ ub,
                                                   float* __restrict__ beta, float* __restrict__ eb,
                                                   float* __restrict__ y, int K, int N, int Kp, int Np) {
  __shared__ float part[16][64];
  const int cq = threadIdx.x & 15, rg = threadIdx.x >> 4;
  const int cblocks = Np / 64;
  const long batch = blockIdx.x / cblocks;
  const int n = (blockIdx.x - batch * cblocks) * 64 + cq * 4;
  const int cnt = N - n;  // live columns of this lane's four (<= 0: none)
  const elem_t* bc = b + batch * K * N + (cnt > 0 ? n : 0);
  const elem_t* uc = ub ? ub + batch * K * N + (cnt > 0 ? n : 0) : nullptr;
  float4 mx = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
  for (int k = rg; k < K; k += 16) {
    const float4 v = ld4m(bc + (long)k * N, cnt, -INFINITY);
    mx = make_float4(fmaxf(mx.x, v.x), fmaxf(mx.y, v.y), fmaxf(mx.z, v.z), fmaxf(mx.w, v.w));
  }
  st4a(&part[rg][cq * 4], mx);
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float4 v = ld4a(&part[r][cq * 4]);
    mx = make_float4(fmaxf(mx.x, v.x), fmaxf(mx.y, v.y), fmaxf(mx.z, v.z), fmaxf(mx.w, v.w));
  }
  if (rg == 0)
    st4(beta + batch * Np + n, make_float4(cnt > 0 ? mx.x : 0.f, cnt > 1 ? mx.y : 0.f, cnt > 2 ? mx.z : 0.f,
                                           cnt > 3 ? mx.w : 0.f));
  float* ec = eb + batch * Kp * Np + n;
  float* yc = y + batch * Kp * Np + n;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int k = rg; k < Kp; k += 16) {
    const bool in = cnt > 0 && k < K;
    float4 e = zero;
    if (in) {
      const float4 v = ld4m(bc + (long)k * N, cnt, -INFINITY);
      e = make_float4(exp_st(v.x - mx.x), cnt > 1 ? exp_st(v.y - mx.y) : 0.f, cnt > 2 ? exp_st(v.z - mx.z) : 0.f,
                      cnt > 3 ? exp_st(v.w - mx.w) : 0.f);
    }
    st4(ec + (long)k * Np, e);
    st4(yc + (long)k * Np, (uc && in) ? mul4(e, ld4m(uc + (long)k * N, cnt, 0.f)) : zero);
  }
}

// R = exp(alpha + beta - out), H = g R over the padded (Mp, Np) grid (zeros in the padding), four
// cells of a row per lane; an item with a cell beyond the guard is flagged.
__global__ __launch_bounds__(256) void k_bb_prep_h(const elem_t* __restrict__ out, const elem_t* __restrict__ g,
                                                   const float* __restrict__ alpha, const float* __restrict__ beta,
                                                   float* __restrict__ r, float* __restrict__ h,
                                                   int* __restrict__ flags, int M, int N, int Mp, int Np,
                                                   long quads) {
  const long q = (long)blockIdx.x * 256 + threadIdx.x;
  if (q >= quads) return;
  const int nq = Np / 4;
  const int n = (int)(q % nq) * 4;
  const long bm = q / nq;
  const long batch = bm / Mp;
  const int m = (int)(bm - batch * Mp);
  float rv[4] = {0.f, 0.f, 0.f, 0.f}, hv[4] = {0.f, 0.f, 0.f, 0.f};
  const int cnt = N - n;
  if (m < M && cnt > 0) {
    const long src = (batch * M + m) * N + n;
    const float al = alpha[bm];
    const float4 be4 = ld4(beta + batch * Np + n), o4 = ld4m(out + src, cnt, 0.f), g4 = ld4m(g + src, cnt, 0.f);
    const float be[4] = {be4.x, be4.y, be4.z, be4.w}, o[4] = {o4.x, o4.y, o4.z, o4.w}, gv[4] = {g4.x, g4.y, g4.z, g4.w};
    const float lim = kMfmaGuardBits * kLn2 + 1e-3f;
    bool bad = !(al > -INFINITY);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < cnt) {
        const float ex = al + be[i] - o[i];
        // (a negated comparison: NaN and +inf fail it; alpha, beta not finite make ex not finite or NaN)
        bad = bad || !(ex <= lim) || !(be[i] > -INFINITY);
        rv[i] = exp_st(ex);
        hv[i] = gv[i] * rv[i];
      }
    if (bad) flags[batch] = 1;
  }
  st4(r + bm * Np + n, make_float4(rv[0], rv[1], rv[2], rv[3]));
  st4(h + bm * Np + n, make_float4(hv[0], hv[1], hv[2], hv[3]));
}

// One tile of C = P1 Q1 (+ P2 Q2) and its epilogue.  Operands are padded workspace arrays:
//   RT: the rows operand is stored [row][red] (staged transposed), else [red][row];
//   CT: the columns operand is stored [col][red], else [red][col].
constexpr int kEpiRaw = 0, kEpiT = 1, kEpiGrad = 2;
struct BBMM {
  const float* rows[2];
  const float* cols[2];
  int pairs;
  int Rp, Cp, Qp;       // padded extents: output rows, output columns, reduction
  // epilogue
  float* raw;           // kEpiRaw: (B, Rp, Cp)
  const float* f_acc;   // kEpiT: R; kEpiGrad: EA / EB - the factor of the accumulator
  const float* f1;      // kEpiGrad: X / Y or NULL ...
  const float* f2;      //           ... times Ga0 / Gb0, added
  const float* h;       // kEpiT: H
  float* nht;           // kEpiT: -H t
  float* tt;            // kEpiT: t unrounded, (B, R, C) unpadded
  elem_t* dst;          // kEpiT: grad_g; kEpiGrad: grad_a / grad_b; (B, R, C) unpadded
  int R, C;             // true extents of the output
};

template <bool RT, bool CT, int EPI>
__global__ __launch_bounds__(256) void k_bb_mm(const BBMM p) {
  using T = MTile<128, 128>;
  constexpr int NT = T::NT, LDR = T::LDR, LDC = T::LDC;
  using SR = std::conditional_t<RT, StageT<T::TR, NT, LDR>, StageS<T::TR, NT, LDR>>;
  using SC = std::conditional_t<CT, StageT<T::TC, NT, LDC>, StageS<T::TC, NT, LDC>>;
  __shared__ __attribute__((aligned(16))) float smem[2 * kMS * (LDR + LDC)];
  static_assert(2 * kMS * (LDR + LDC) >= (NT / 64) * kStripFloats, "");
  float(*Rs)[kMS * LDR] = reinterpret_cast<float(*)[kMS * LDR]>(smem);
  float(*Cs)[kMS * LDC] = reinterpret_cast<float(*)[kMS * LDC]>(smem + 2 * kMS * LDR);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr0 = (wave / T::WC) * 64, wc0 = (wave % T::WC) * 64;
  const int tiles_c = p.Cp / T::TC, per = (p.Rp / T::TR) * tiles_c;
  const int tile = xcd_tile_id();
  const int batch = tile / per, rem = tile - batch * per;
  const int r0 = (rem / tiles_c) * T::TR, c0 = (rem % tiles_c) * T::TC;
  const int Qp = p.Qp, slabs = Qp / kMS;

  floatx16 acc[2][2];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[x >> 1][x & 1][i] = 0.f;

  for (int pair = 0; pair < p.pairs; ++pair) {
    const float* pr[SR::PER];
    const float* pc[SC::PER];
    const float* rbase = p.rows[pair] + (long)batch * p.Rp * Qp;
    const float* cbase = p.cols[pair] + (long)batch * p.Cp * Qp;
#pragma unroll
    for (int l = 0; l < SR::PER; ++l) {
      if constexpr (RT) pr[l] = rbase + (long)(r0 + SR::line(tid, l)) * Qp + SR::quad(tid) * 4;
      else pr[l] = rbase + (long)SR::red(tid, l) * p.Rp + r0 + SR::quad(tid) * 4;
    }
#pragma unroll
    for (int l = 0; l < SC::PER; ++l) {
      if constexpr (CT) pc[l] = cbase + (long)(c0 + SC::line(tid, l)) * Qp + SC::quad(tid) * 4;
      else pc[l] = cbase + (long)SC::red(tid, l) * p.Cp + c0 + SC::quad(tid) * 4;
    }
    float4 rr[SR::PER], rc[SC::PER];
    auto load = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int l = 0; l < SR::PER; ++l) {
        rr[l] = ld4a(pr[l]);
        pr[l] += RT ? (long)kMS : (long)kMS * p.Rp;
      }
#pragma unroll
      for (int l = 0; l < SC::PER; ++l) {
        rc[l] = ld4a(pc[l]);
        pc[l] += CT ? (long)kMS : (long)kMS * p.Cp;
      }
    };
    auto stage = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
      for (int l = 0; l < SR::PER; ++l) SR::put(Rs[buf], tid, l, rr[l]);
#pragma unroll
      for (int l = 0; l < SC::PER; ++l) SC::put(Cs[buf], tid, l, rc[l]);
    };
    load();
    stage(0);
    __syncthreads();
    for (int s = 0; s < slabs; ++s) {
      const bool more = s + 1 < slabs;
      if (more) load();
      mfma_slab<LDR, LDC>(Rs[s & 1], Cs[s & 1], wr0, wc0, lane, acc);
      if (more) stage((s + 1) & 1);
      __syncthreads();
    }
  }

  // epilogue, row-wise: f(q, t, v) = four columns lc .. lc + 3 of block row 16 q + 4 t + lr
  const int lr = lane >> 4, lc = (lane & 15) * 4;
  const int row0 = r0 + wr0 + lr, col = c0 + wc0 + lc;
  const long pbase = ((long)batch * p.Rp + row0) * p.Cp + col;   // padded arrays
  const int cc = clamp4(p.C - col);                              // columns of the piece that exist
  acc_rows(acc, smem + wave * kStripFloats, lane, [](int) {},
           [&](int q, int t, float4 v) __attribute__((always_inline)) {
             const int ru = 16 * q + 4 * t;
             const long pu = pbase + (long)ru * p.Cp;
             const bool live = row0 + ru < p.R && cc > 0;
             const long du = ((long)batch * p.R + row0 + ru) * p.C + col;  // unpadded arrays
             if constexpr (EPI == kEpiRaw) {
               st4a(p.raw + pu, v);
             } else if constexpr (EPI == kEpiT) {
               const float4 rv = ld4a(p.f_acc + pu), hv = ld4a(p.h + pu);
               const float4 tv = make_float4(rv.x * v.x, rv.y * v.y, rv.z * v.z, rv.w * v.w);
               st4a(p.nht + pu, make_float4(-hv.x * tv.x, -hv.y * tv.y, -hv.z * tv.z, -hv.w * tv.w));
               if (live) {
                 st4m(p.tt + du, cc, tv);
                 if constexpr (!kElemF32) st4m(p.dst + du, cc, tv);
               }
             } else {
               const float4 fa = ld4a(p.f_acc + pu);
               float4 o = make_float4(fa.x * v.x, fa.y * v.y, fa.z * v.z, fa.w * v.w);
               if (p.f1) {
                 const float4 x1 = ld4a(p.f1 + pu), x2 = ld4a(p.f2 + pu);
                 o = make_float4(__builtin_fmaf(x1.x, x2.x, o.x), __builtin_fmaf(x1.y, x2.y, o.y),
                                 __builtin_fmaf(x1.z, x2.z, o.z), __builtin_fmaf(x1.w, x2.w, o.w));
               }
               if (live) st4m(p.dst + du, cc, o);
             }
           });
}

template <bool RT, bool CT, int EPI>
int launch_mm(const BBMM& p, int B, hipStream_t s) {
  const int64_t tiles = (int64_t)B * (p.Rp / 128) * (p.Cp / 128);
  if (tiles > 0x7fffffffLL) return GENBMM_E_SHAPE;
  hipLaunchKernelGGL((k_bb_mm<RT, CT, EPI>), dim3((unsigned)tiles), dim3(256), 0, s, p);
  return launch_status();
}

int bwdbwd_factored(const BB& p, const BBWs& w, int B, hipStream_t s) {
  const int M = p.M, K = p.K, N = p.N, Mp = bb_pad(M), Kp = bb_pad(K), Np = bb_pad(N);
  {
    const long rows = (long)B * Mp;
    const long per_wg = Kp == 128 ? 8 : 4;  // rows per workgroup: 32 or 64 lanes each
    hipLaunchKernelGGL(k_bb_prep_a, dim3((unsigned)((rows + per_wg - 1) / per_wg)), dim3(256), 0, s, p.a, p.ua, w.alpha, w.ea,
                       w.x, w.flags, M, K, Mp, Kp, rows);
    hipLaunchKernelGGL(k_bb_prep_b, dim3((unsigned)(B * (Np / 64))), dim3(256), 0, s, p.b, p.ub, w.beta, w.eb, w.y,
                       K, N, Kp, Np);
    const long quads = (long)B * Mp * (Np / 4);
    hipLaunchKernelGGL(k_bb_prep_h, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, p.out, p.g, w.alpha,
                       w.beta, w.r, w.h, w.flags, M, N, Mp, Np, quads);
    if (int e = launch_status()) return e;
  }
  const bool has_a = p.ua != nullptr, has_b = p.ub != nullptr;
  {  // t = R (X EB + EA Y); also -H t and grad_g
    BBMM q{};
    int n = 0;
    if (has_a) { q.rows[n] = w.x; q.cols[n] = w.eb; ++n; }
    if (has_b) { q.rows[n] = w.ea; q.cols[n] = w.y; ++n; }
    q.pairs = n; q.Rp = Mp; q.Cp = Np; q.Qp = Kp; q.R = M; q.C = N;
    q.f_acc = w.r; q.h = w.h; q.nht = w.nht; q.tt = p.tt; q.dst = p.gg;
    if (int e = launch_mm<true, false, kEpiT>(q, B, s)) return e;
  }
  if (has_a) {  // Ga0 = H EB^T
    BBMM q{};
    q.rows[0] = w.h; q.cols[0] = w.eb; q.pairs = 1;
    q.Rp = Mp; q.Cp = Kp; q.Qp = Np; q.R = M; q.C = K; q.raw = w.ga0;
    if (int e = launch_mm<true, true, kEpiRaw>(q, B, s)) return e;
  }
  {  // grad_a = X Ga0 + EA (H Y^T - (H t) EB^T)
    BBMM q{};
    int n = 0;
    if (has_b) { q.rows[n] = w.h; q.cols[n] = w.y; ++n; }
    q.rows[n] = w.nht; q.cols[n] = w.eb; ++n;
    q.pairs = n; q.Rp = Mp; q.Cp = Kp; q.Qp = Np; q.R = M; q.C = K;
    q.f_acc = w.ea; q.f1 = has_a ? w.x : nullptr; q.f2 = w.ga0; q.dst = p.ga;
    if (int e = launch_mm<true, true, kEpiGrad>(q, B, s)) return e;
  }
  if (has_b) {  // Gb0 = EA^T H
    BBMM q{};
    q.rows[0] = w.ea; q.cols[0] = w.h; q.pairs = 1;
    q.Rp = Kp; q.Cp = Np; q.Qp = Mp; q.R = K; q.C = N; q.raw = w.gb0;
    if (int e = launch_mm<false, false, kEpiRaw>(q, B, s)) return e;
  }
  {  // grad_b = Y Gb0 + EB (X^T H - EA^T (H t))
    BBMM q{};
    int n = 0;
    if (has_a) { q.rows[n] = w.x; q.cols[n] = w.h; ++n; }
    q.rows[n] = w.ea; q.cols[n] = w.nht; ++n;
    q.pairs = n; q.Rp = Kp; q.Cp = Np; q.Qp = Mp; q.R = K; q.C = N;
    q.f_acc = w.eb; q.f1 = has_b ? w.y : nullptr; q.f2 = w.gb0; q.dst = p.gb;
    if (int e = launch_mm<false, false, kEpiGrad>(q, B, s)) return e;
  }
  // items beyond the guard: the exact passes, on those items only
  BB ex = p;
  ex.only = w.flags;
  return launch_exact(ex, B, s);
}

int bwdbwd(const elem_t* a, const elem_t* b, const elem_t* out, const elem_t* g, const elem_t* u_a,
           const elem_t* u_b, elem_t* grad_a, elem_t* grad_b, elem_t* grad_g, float* workspace, int B, int M,
           int K, int N, void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  {
    const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
    if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(g, mn) ||
        missing(grad_a, mk) || missing(grad_b, kn) || missing(grad_g, mn) ||
        (missing(u_a, mk) && missing(u_b, kn)))
      return GENBMM_E_NULLPTR;
    if (!kElemF32 && missing(workspace, mn)) return GENBMM_E_NULLPTR;  // t must stay unrounded somewhere
  }
  hipStream_t s = (hipStream_t)stream;
  BB p{a, b, out, g, u_a, u_b, grad_a, grad_b, grad_g, nullptr, nullptr, M, K, N, B};
  BBWs w{};
  if (workspace) bb_ws_floats(B, M, K, N, &w, workspace);
  if constexpr (kElemF32) p.tt = reinterpret_cast<float*>(grad_g);
  else p.tt = w.t_exact;
  if (workspace && bb_factored_ok(B, M, K, N) && (int64_t)B * M * K > 0 && (int64_t)B * K * N > 0)
    return bwdbwd_factored(p, w, B, s);
  return launch_exact(p, B, s);
}

}  // namespace
}  // namespace GENBMM_NS

extern "C" {

#if GENBMM_ELEM == 0
size_t genbmm_logbmm_bwdbwd_ws_size(int B, int M, int K, int N) {
  using namespace GENBMM_NS;
  if (check_dense_dims(B, M, K, N)) return 0;
  return bb_ws_floats(B, M, K, N, nullptr, nullptr);
}

int genbmm_logbmm_bwdbwd(const float* a, const float* b, const float* out, const float* g,
                         const float* u_a, const float* u_b, float* grad_a, float* grad_b,
                         float* grad_g, int B, int M, int K, int N, void* stream) {
  return GENBMM_NS::bwdbwd(a, b, out, g, u_a, u_b, grad_a, grad_b, grad_g, nullptr, B, M, K, N, stream);
}
#endif

// One per element type: genbmm_logbmm_bwdbwd_ws, ..._ws_f16, ..._ws_bf16
int GENBMM_API(logbmm_bwdbwd_ws)(const GENBMM_NS::abi_t* a, const GENBMM_NS::abi_t* b, const GENBMM_NS::abi_t* out,
                                 const GENBMM_NS::abi_t* g, const GENBMM_NS::abi_t* u_a, const GENBMM_NS::abi_t* u_b,
                                 GENBMM_NS::abi_t* grad_a, GENBMM_NS::abi_t* grad_b, GENBMM_NS::abi_t* grad_g,
                                 float* workspace, int B, int M, int K, int N, void* stream) {
  using namespace GENBMM_NS;
  return bwdbwd(el(a), el(b), el(out), el(g), el(u_a), el(u_b), el(grad_a), el(grad_b), el(grad_g), workspace, B, M, K,
                N, stream);
}

}  // extern "C"
