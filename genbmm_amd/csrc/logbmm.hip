// logbmm forward and backward (gfx950): the exact online-log-sum-exp kernels and
// the factored kernels that replace the per-element exponential by one fused
// multiply-add whenever that is provably as accurate.
//
// Factored form.  With row/column shifts alpha[m] = max_k a[m,k] and
// beta[n] = max_k b[k,n] (the "stats" vector, alpha then beta per batch item):
//
//   EA[m,k] = exp(a[m,k] - alpha[m])  in (0,1]     EB[k,n] = exp(b[k,n] - beta[n])
//   S[m,n]  = sum_k EA[m,k] * EB[k,n]              out = log S + alpha + beta
//   H[m,n]  = g[m,n] * exp(alpha[m] + beta[n] - out[m,n])            ( = g / S )
//   grad_a[m,k] = EA[m,k] * sum_n H[m,n] * EB[k,n]
//   grad_b[k,n] = EB[k,n] * sum_m EA[m,k] * H[m,n]
//
// The exponentials are taken while a tile is staged into LDS (once per tile
// element, not once per (m,k,n)), the contraction itself is v_fma_f32 on
// register blocks.  A factor can only underflow for a term that is below
// 2^-126 of the bound exp(alpha+beta); as long as S >= 2^-40 such terms are
// below 2^-86 of the result, i.e. invisible in fp32.  Each workgroup checks that
// condition for its own tile (forward: on S; backward: on alpha+beta-out while
// staging H) and, if any cell fails it - or is NaN/inf, or sits at the
// reference's -1e9 floor - raises that tile's flag instead of storing; a fix-up
// kernel launched right behind recomputes exactly the flagged tiles with the
// exact kernel's routine (online running-max log-sum-exp forward, exp(a+b-out)
// backward), so the result never depends on the factoring being applicable.
// The flags live behind the shifts in the caller's `stats` buffer.
//
// Two implementations of the factored contraction: v_fma_f32 on register blocks
// (any shape, this file) and the fp32 matrix-core instruction for problems made
// of full 128x128 tiles (logbmm_mfma.h).
#include <algorithm>
#include <mutex>

#include "dense_tiles.h"
#include "log_bwd_tile.h"
#include "logbmm_item.h"
#include "logbmm_mfma.h"
#include "logbmm_split.h"
#include "logbmm_item32.h"
#include "logbmm_self.h"
#include "logbmm_ws.h"

namespace GENBMM_NS {
namespace {

constexpr float kLog2eLo = 1.92596299e-8f;  // log2(e) - (float)log2(e)
constexpr float kGuardBits = 40.f;          // factored path needs S >= 2^-40

// exp(d) for staged tile elements: one multiply and v_exp_f32.  The rounding of
// d*log2e costs |d| * 6e-8 relative; terms that matter have |d| < ~28 (guard).
__device__ __forceinline__ float exp_stage(float d) { return fast_exp2(d * kLog2e); }

// exp(d) through v_exp_f32 with the rounding error of d*log2e compensated
// (used once per output element).
__device__ __forceinline__ float exp_comp(float d) {
  const float hi = d * kLog2e;
  const float lo = __builtin_fmaf(d, kLog2e, -hi) + d * kLog2eLo;
  const float e = fast_exp2(hi);
  // (d = -inf, a masked entry: hi - hi is NaN in `lo`; the result is the plain 0)
  return hi == -INFINITY ? 0.f : __builtin_fmaf(e, lo * kLn2, e);
}

// ------------------------------------------------------------------ stats
// stats[b][0..M) = max_k a[b,m,k],  stats[b][M..M+N) = max_k b[b,k,n].
// Workgroups [0, row_wgs) of a batch item take kStatRows rows of a each (a wave
// owns four rows and keeps their loads in flight together); the remaining
// col_wgs take kStatCols columns of b each (8 float4 lanes across, 32 row
// groups down, reduced through LDS).
constexpr int kStatRows = 16, kStatCols = 32;

__global__ __launch_bounds__(256) void k_log_stats(const elem_t* __restrict__ a,
                                                   const elem_t* __restrict__ b,
                                                   float* __restrict__ stats, int* __restrict__ hdr,
                                                   int M, int K, int N, int row_wgs, int col_wgs,
                                                   int vec_a, int vec_b) {
  __shared__ float part[32][kStatCols + 1];
  if (blockIdx.x == 0 && threadIdx.x == 0) hdr[0] = 0;  // by-products of an earlier forward are stale
  const int per = row_wgs + col_wgs;
  const int batch = blockIdx.x / per;
  const int wg = blockIdx.x - batch * per;
  const int tid = threadIdx.x;
  float* st = stats + (long)batch * (M + N);
  if (wg < row_wgs) {
    const int lane = tid & 63, m0 = wg * kStatRows + (tid >> 6) * 4;
    const elem_t* base = a + ((long)batch * M + m0) * K;
    float v[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    if (vec_a && m0 + 3 < M) {
      for (int k = lane * 4; k < K; k += 256) {
        float4 x[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) x[r] = ld4a(base + (long)r * K + k);
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = fmaxf(v[r], fmaxf(fmaxf(x[r].x, x[r].y), fmaxf(x[r].z, x[r].w)));
      }
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (m0 + r < M)
          for (int k = lane; k < K; k += 64) v[r] = fmaxf(v[r], base[(long)r * K + k]);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) v[r] = fmaxf(v[r], __shfl_xor(v[r], off, 64));
      if (lane == 0 && m0 + r < M) st[m0 + r] = v[r];
    }
  } else {
    const int c4 = tid & 7, rg = tid >> 3;
    const int n = (wg - row_wgs) * kStatCols + c4 * 4;
    const elem_t* col = b + (long)batch * K * N + n;
    float4 v = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    if (n < N) {
      if (vec_b) {
        int k = rg;
        for (; k + 96 < K; k += 128) {  // four rows in flight
          float4 x[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) x[r] = ld4a(col + (long)(k + 32 * r) * N);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            v.x = fmaxf(v.x, x[r].x); v.y = fmaxf(v.y, x[r].y);
            v.z = fmaxf(v.z, x[r].z); v.w = fmaxf(v.w, x[r].w);
          }
        }
        for (; k < K; k += 32) {
          const float4 x = ld4a(col + (long)k * N);
          v.x = fmaxf(v.x, x.x); v.y = fmaxf(v.y, x.y); v.z = fmaxf(v.z, x.z); v.w = fmaxf(v.w, x.w);
        }
      } else {
        for (int k = rg; k < K; k += 32) {
          const elem_t* p = col + (long)k * N;
          v.x = fmaxf(v.x, p[0]);
          if (n + 1 < N) v.y = fmaxf(v.y, p[1]);
          if (n + 2 < N) v.z = fmaxf(v.z, p[2]);
          if (n + 3 < N) v.w = fmaxf(v.w, p[3]);
        }
      }
    }
    part[rg][c4 * 4 + 0] = v.x; part[rg][c4 * 4 + 1] = v.y;
    part[rg][c4 * 4 + 2] = v.z; part[rg][c4 * 4 + 3] = v.w;
    __syncthreads();
    if (tid < kStatCols) {
      const int nn = (wg - row_wgs) * kStatCols + tid;
      if (nn < N) {
        float r = part[0][tid];
#pragma unroll
        for (int q = 1; q < 32; ++q) r = fmaxf(r, part[q][tid]);
        st[M + nn] = r;
      }
    }
  }
}

// The same maxima for a problem with few rows and columns and a long K, where the kernel above
// would walk all of K in a handful of workgroups: the reduction axis in parts, a workgroup per
// batch item, part and operand, joined by an integer atomic on the bit pattern (max of the
// pattern for values >= 0, min for negative ones - the order of floats), which commutes: the
// result is the kernel above's whatever order the parts arrive in.  k_log_stats_init fills the
// maxima with -inf first.
__global__ __launch_bounds__(256) void k_log_stats_init(float* __restrict__ stats, int* __restrict__ hdr, long count) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e < count) stats[e] = -INFINITY;
  if (e == 0) hdr[0] = 0;  // by-products of an earlier forward are stale
}
__device__ __forceinline__ void stat_join(float* __restrict__ at, float v) {
  v += 0.f;  // -0 joins as +0
  if (v >= 0.f) atomicMax(reinterpret_cast<int*>(at), __float_as_int(v));
  else if (v > -INFINITY) atomicMin(reinterpret_cast<unsigned*>(at), __float_as_uint(v));
}
__global__ __launch_bounds__(256) void k_log_stats_parts(const elem_t* __restrict__ a, const elem_t* __restrict__ b,
                                                        float* __restrict__ stats, int M, int K, int N, int kparts,
                                                        int klen) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rows = blockIdx.x & 1, part = (blockIdx.x >> 1) % kparts, batch = (blockIdx.x >> 1) / kparts;
  const int k0 = part * klen, k1 = min(K, k0 + klen);
  float* st = stats + (long)batch * (M + N);
  if (rows) {  // a wave per row, its lanes along k
    for (int m = wave; m < M; m += 4) {
      const elem_t* row = a + ((long)batch * M + m) * K;
      float v = -INFINITY;
      for (int k = k0 + lane; k < k1; k += 64) v = fmaxf(v, (float)row[k]);
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
      if (lane == 0) stat_join(st + m, v);
    }
  } else {  // lanes along n, the waves take every fourth k
    for (int n0 = 0; n0 < N; n0 += 64) {
      const int n = n0 + lane;
      if (n >= N) continue;
      const elem_t* col = b + (long)batch * K * N + n;
      float v = -INFINITY;
      int k = k0 + wave;
      for (; k + 12 < k1; k += 16) {  // four rows in flight
        const float x0 = col[(long)k * N], x1 = col[(long)(k + 4) * N], x2 = col[(long)(k + 8) * N], x3 = col[(long)(k + 12) * N];
        v = fmaxf(fmaxf(fmaxf(fmaxf(v, x0), x1), x2), x3);  // (each maximum against the float: none narrows to the element type)
      }
      for (; k < k1; k += 4) v = fmaxf(v, (float)col[(long)k * N]);
      stat_join(st + M + n, v);
    }
  }
}

// ------------------------------------------------------------ exact kernels
template <class C>
__global__ __launch_bounds__(C::NT) void k_log_fwd_exact(const DenseArgs p) {
  __shared__ __attribute__((aligned(16))) float smem[C::KT * (C::LDA + C::LDB)];
  int batch, m0, n0;
  decode_tile<C>(p, batch, m0, n0);
  log_fwd_tile<C, false>(p, batch, m0, n0, smem, smem + C::KT * C::LDA);
}

template <class C, bool GRAD_A>
__global__ __launch_bounds__(C::NT) void k_log_bwd_exact(const LogBwdArgs p) {
  __shared__ __attribute__((aligned(16))) float smem[LogBwdLds<C, GRAD_A>::FLOATS];
  const int per = p.tiles_r * p.tiles_c;
  const int tile = xcd_renumber(blockIdx.x, gridDim.x);
  const int batch = tile / per;
  const int rem = tile - batch * per;
  log_bwd_tile<C, GRAD_A>(p, batch, (rem / p.tiles_c) * C::BR, (rem % p.tiles_c) * C::BC, smem);
}

// --------------------------------------------------------- factored forward
template <class C>
__global__ __launch_bounds__(C::NT, 2) void k_log_fwd_fast(const DenseArgs p,
                                                           const float* __restrict__ stats,
                                                           int* __restrict__ flags,
                                                           int* __restrict__ hdr) {
  __shared__ __attribute__((aligned(16))) float smem[C::KT * (C::LDA + C::LDB) + C::BM + C::BN];
  float* As = smem;
  float* Bs = As + C::KT * C::LDA;
  float* al = Bs + C::KT * C::LDB;
  float* be = al + C::BM;
  const int tid = threadIdx.x, tx = tid % C::TX, ty = tid / C::TX;
  int batch, m0, n0;
  decode_tile<C>(p, batch, m0, n0);
  const int M = p.M, K = p.K, N = p.N;
  if (blockIdx.x == 0 && tid == 0) {  // whose flags these are, and their tile shape
    hdr[1] = C::BM;
    hdr[2] = C::BN;
    hdr[0] = kWsFast;
  }
  const elem_t* ab = p.a + (long)batch * M * K;
  const elem_t* bb = p.b + (long)batch * K * N;
  const float* st = stats + (long)batch * (M + N);
  for (int t = tid; t < C::BM; t += C::NT) al[t] = (m0 + t < M) ? st[m0 + t] : 0.f;
  for (int t = tid; t < C::BN; t += C::NT) be[t] = (n0 + t < N) ? st[M + n0 + t] : 0.f;
  __syncthreads();

  float acc[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j) acc[i][j] = 0.f;

  using TA = TileOutMajor<C::BM, C::KT, C::NT>;
  using TB = TileRedMajor<C::BN, C::KT, C::NT>;
  TA ta;
  TB tb;
  if (K > 0) {
    ta.gload(ab, K, m0, 0, M, K, p.vec_a, tid);
    tb.gload(bb, N, n0, 0, N, K, p.vec_b, tid);
  }
  for (int k0 = 0; k0 < K; k0 += C::KT) {
    __syncthreads();
#pragma unroll
    for (int l = 0; l < TA::PER; ++l) {  // EA = exp(a - alpha[row])
      const float s = al[((tid + l * C::NT) / TA::C4) % C::BM];
      ta.r[l].x = exp_stage(ta.r[l].x - s); ta.r[l].y = exp_stage(ta.r[l].y - s);
      ta.r[l].z = exp_stage(ta.r[l].z - s); ta.r[l].w = exp_stage(ta.r[l].w - s);
    }
#pragma unroll
    for (int l = 0; l < TB::PER; ++l) {  // EB = exp(b - beta[col])
      const float4 s = *reinterpret_cast<const float4*>(be + ((tid + l * C::NT) % TB::C4) * 4);
      tb.r[l].x = exp_stage(tb.r[l].x - s.x); tb.r[l].y = exp_stage(tb.r[l].y - s.y);
      tb.r[l].z = exp_stage(tb.r[l].z - s.z); tb.r[l].w = exp_stage(tb.r[l].w - s.w);
    }
    ta.sstore(As, tid);
    tb.sstore(Bs, tid);
    __syncthreads();
    if (k0 + C::KT < K) {
      ta.gload(ab, K, m0, k0 + C::KT, M, K, p.vec_a, tid);
      tb.gload(bb, N, n0, k0 + C::KT, N, K, p.vec_b, tid);
    }
    const int kn = min(C::KT, K - k0);
    auto step = [&](int kk) __attribute__((always_inline)) {
      float av[C::TM], bv[C::TN];
      lds_frag<C::TM / 4>(As + kk * C::LDA, ty * C::TM, 4, av);
      lds_frag<C::TN / 4>(Bs + kk * C::LDB, tx * 4, C::TX * 4, bv);
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j) acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
    };
    if (kn == C::KT) {
#pragma unroll 2
      for (int kk = 0; kk < C::KT; ++kk) step(kk);
    } else {
      for (int kk = 0; kk < kn; ++kk) step(kk);
    }
  }

  // guard + epilogue
  const float thr = __builtin_amdgcn_exp2f(-kGuardBits);
  int bad = 0;
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
    const int r = ty * C::TM + i;
    const float ai = al[r];
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
      const int c = col_of<C>(tx, j);
      const float shift = ai + be[c];
      const float s = acc[i][j];
      const bool ok = (s >= thr) && (s < INFINITY) && (shift >= kFloor) && (shift < INFINITY);
      if (!ok && m0 + r < M && n0 + c < N) bad = 1;
      acc[i][j] = __builtin_fmaf(fast_log2(s), kLn2, shift);  // v_log_f32
    }
  }
  bad = __syncthreads_or(bad);
  if (tid == 0) flags[xcd_renumber(blockIdx.x, gridDim.x)] = bad;  // the tile's number, as decode_tile has it
  if (bad) return;  // the fix-up launch recomputes this tile
  store_tile_f<C>(p.out + (long)batch * M * N, acc, m0, n0, M, N, p.vec_o, tx, ty);
}

// Recompute the flagged tiles of a factored forward launch with the online
// routine.  FBM x FBN is the factored launch's tile, CX the exact routine's
// tile (which divides it).  Workgroups stride over the tile list.
template <class CX, int FBM, int FBN>
__global__ __launch_bounds__(CX::NT) void k_log_fwd_fixup(const DenseArgs p,
                                                          const int* __restrict__ flags,
                                                          int total_tiles) {
  static_assert(FBM % CX::BM == 0 && FBN % CX::BN == 0, "");
  __shared__ __attribute__((aligned(16))) float smem[CX::KT * (CX::LDA + CX::LDB)];
  const int per = p.tiles_m * p.tiles_n;  // of the factored launch
  for (int t = blockIdx.x; t < total_tiles; t += gridDim.x) {
    if (!flags[t]) continue;
    const int batch = t / per, r = t - batch * per;
    const int m0 = (r / p.tiles_n) * FBM, n0 = (r % p.tiles_n) * FBN;
    for (int h = 0; h < FBM / CX::BM; ++h)
      for (int w = 0; w < FBN / CX::BN; ++w)
        if (m0 + h * CX::BM < p.M && n0 + w * CX::BN < p.N) {
          log_fwd_tile<CX, false>(p, batch, m0 + h * CX::BM, n0 + w * CX::BN, smem,
                                  smem + CX::KT * CX::LDA);
          __syncthreads();
        }
  }
}

// The same for samplebmm: log-sum-exp and index of the flagged tiles by the exact walk.
template <class CX, int FBM, int FBN>
__global__ __launch_bounds__(CX::NT) void k_sample_fixup(const DenseArgs p,
                                                         const int* __restrict__ flags,
                                                         int total_tiles) {
  static_assert(FBM % CX::BM == 0 && FBN % CX::BN == 0, "");
  __shared__ __attribute__((aligned(16))) float smem[CX::KT * (CX::LDA + CX::LDB)];
  const int per = p.tiles_m * p.tiles_n;
  for (int t = blockIdx.x; t < total_tiles; t += gridDim.x) {
    if (!flags[t]) continue;
    const int batch = t / per, r = t - batch * per;
    const int m0 = (r / p.tiles_n) * FBM, n0 = (r % p.tiles_n) * FBN;
    for (int h = 0; h < FBM / CX::BM; ++h)
      for (int w = 0; w < FBN / CX::BN; ++w)
        if (m0 + h * CX::BM < p.M && n0 + w * CX::BN < p.N) {
          log_fwd_tile<CX, true>(p, batch, m0 + h * CX::BM, n0 + w * CX::BN, smem,
                                 smem + CX::KT * CX::LDA);
          __syncthreads();
        }
  }
}

// Backward fix-up: recompute, with the exact routine, the tiles of a factored backward
// launch that left their work undone.  Whether a tile did is a function of what the
// forward left in the workspace (bwd_tile_flagged), evaluated here exactly as in the
// launch itself; the workspace is only read.
template <class CX, int FBR, int FBC, bool GRAD_A>
__global__ __launch_bounds__(CX::NT) void k_log_bwd_fixup(const LogBwdArgs p,
                                                          const int* __restrict__ hdr,
                                                          const int* __restrict__ fwd_flags,
                                                          int need_factors, int total_tiles) {
  static_assert(FBR % CX::BR == 0 && FBC % CX::BC == 0, "");
  __shared__ __attribute__((aligned(16))) float smem[LogBwdLds<CX, GRAD_A>::FLOATS];
  const int per = p.tiles_r * p.tiles_c;  // of the factored launch
  const int R = GRAD_A ? p.M : p.K, Cc = GRAD_A ? p.K : p.N;
  for (int t = blockIdx.x; t < total_tiles; t += gridDim.x) {
    const int batch = t / per, r = t - batch * per;
    const int r0 = (r / p.tiles_c) * FBR, c0 = (r % p.tiles_c) * FBC;
    if (!bwd_tile_flagged(hdr, fwd_flags, need_factors, GRAD_A, GRAD_A ? r0 : c0, GRAD_A ? FBR : FBC,
                          batch, p.M, p.N, threadIdx.x, CX::NT))
      continue;
    for (int h = 0; h < FBR / CX::BR; ++h)
      for (int w = 0; w < FBC / CX::BC; ++w)
        if (r0 + h * CX::BR < R && c0 + w * CX::BC < Cc) {
          log_bwd_tile<CX, GRAD_A>(p, batch, r0 + h * CX::BR, c0 + w * CX::BC, smem);
          __syncthreads();
        }
  }
}

// Fix-up of both gradients' tiles in one launch (workgroups stride over the grad_a
// list, then over the grad_b list).
template <class CX, int AR, int AC, int BR, int BC>
__global__ __launch_bounds__(CX::NT) void k_log_bwd_fixup_both(const LogBwdArgs pa,
                                                               const LogBwdArgs pb,
                                                               const int* __restrict__ hdr,
                                                               const int* __restrict__ fwd_flags,
                                                               int tiles_a, int tiles_b, int need_factors) {
  constexpr int kFa = LogBwdLds<CX, true>::FLOATS, kFb = LogBwdLds<CX, false>::FLOATS;
  __shared__ __attribute__((aligned(16))) float smem[kFa > kFb ? kFa : kFb];
  for (int t = blockIdx.x; t < tiles_a + tiles_b; t += gridDim.x) {
    const bool is_a = t < tiles_a;
    const int u = is_a ? t : t - tiles_a;
    const LogBwdArgs& p = is_a ? pa : pb;
    const int per = p.tiles_r * p.tiles_c;
    const int batch = u / per, r = u - batch * per;
    const int FR = is_a ? AR : BR, FC = is_a ? AC : BC;
    const int R = is_a ? p.M : p.K, Cc = is_a ? p.K : p.N;
    const int r0 = (r / p.tiles_c) * FR, c0 = (r % p.tiles_c) * FC;
    if (!bwd_tile_flagged(hdr, fwd_flags, need_factors, is_a, is_a ? r0 : c0, is_a ? FR : FC, batch, p.M, p.N,
                          threadIdx.x, CX::NT))
      continue;
    for (int h = 0; h < FR / CX::BR; ++h)
      for (int w = 0; w < FC / CX::BC; ++w)
        if (r0 + h * CX::BR < R && c0 + w * CX::BC < Cc) {
          if (is_a) log_bwd_tile<CX, true>(p, batch, r0 + h * CX::BR, c0 + w * CX::BC, smem);
          else log_bwd_tile<CX, false>(p, batch, r0 + h * CX::BR, c0 + w * CX::BC, smem);
          __syncthreads();
        }
  }
}

// -------------------------------------------------------- factored backward
// Output tile (rows r, cols c) = (m,k) for grad_a, (k,n) for grad_b; the
// reduction index q is n or m.  Y = the other operand, staged as exp(y - shift);
// H = g*exp(alpha+beta-out), staged from out and g; X = the operand shaped like
// the output, read once in the epilogue.
template <class C, bool GRAD_A>
__global__ __launch_bounds__(C::NT, 2) void k_log_bwd_fast(const LogBwdArgs p,
                                                           const float* __restrict__ stats,
                                                           const int* __restrict__ hdr,
                                                           const int* __restrict__ fwd_flags) {
  constexpr int BY = GRAD_A ? C::BC : C::BR;
  constexpr int BO = GRAD_A ? C::BR : C::BC;
  using TYt = std::conditional_t<GRAD_A, TileOutMajor<BY, C::RT, C::NT>, TileRedMajor<BY, C::RT, C::NT>>;
  using TOt = std::conditional_t<GRAD_A, TileOutMajor<BO, C::RT, C::NT>, TileRedMajor<BO, C::RT, C::NT>>;
  constexpr int LDY = BY + kPad, LDO = BO + kPad;
  __shared__ __attribute__((aligned(16))) float smem[C::RT * (LDY + LDO)];
  float* Ys = smem;
  float* Hs = smem + C::RT * LDY;

  const int tid = threadIdx.x, tx = tid % C::TX, ty = tid / C::TX;
  const int M = p.M, K = p.K, N = p.N;
  const int R = GRAD_A ? M : K, Cc = GRAD_A ? K : N, Q = GRAD_A ? N : M;
  const int per = p.tiles_r * p.tiles_c;
  const int tile = xcd_renumber(blockIdx.x, gridDim.x);
  const int batch = tile / per;
  const int rem = tile - batch * per;
  const int r0 = (rem / p.tiles_c) * C::BR, c0 = (rem % p.tiles_c) * C::BC;
  // Every cell this tile reduces over must come from a forward tile that passed the
  // factoring guard (S >= 2^-40, finite shifts): H = g * exp(alpha + beta - out) is then
  // at most |g| * 2^40.  Otherwise the fix-up launch recomputes this tile.
  if (bwd_tile_flagged(hdr, fwd_flags, false, GRAD_A, GRAD_A ? r0 : c0, GRAD_A ? C::BR : C::BC, batch, M,
                       N, tid, C::NT))
    return;

  const elem_t* ab = p.a + (long)batch * M * K;
  const elem_t* bb = p.b + (long)batch * K * N;
  const elem_t* ob = p.out + (long)batch * M * N;
  const elem_t* gb = p.g + (long)batch * M * N;
  const elem_t* xb = GRAD_A ? ab : bb;
  const elem_t* yb = GRAD_A ? bb : ab;
  const float* al = stats + (long)batch * (M + N);  // alpha[m]
  const float* be = al + M;                         // beta[n]
  const long ldy = GRAD_A ? N : K;
  const bool vec_x = GRAD_A ? p.vec_k : p.vec_n;
  const bool vec_y = GRAD_A ? p.vec_n : p.vec_k;
  const bool vec_o = p.vec_n;
  const int y0 = GRAD_A ? c0 : r0;
  const int o0 = GRAD_A ? r0 : c0, olim = GRAD_A ? M : N;

  auto col_of = [&](int j) { return (j >> 2) * (C::TX * 4) + tx * 4 + (j & 3); };
  auto safe = [](const float* v, int i, int n) { return i < n ? v[i] : 0.f; };

  float acc[C::TR][C::TC];
#pragma unroll
  for (int i = 0; i < C::TR; ++i)
#pragma unroll
    for (int j = 0; j < C::TC; ++j) acc[i][j] = 0.f;

  // Shifts that do not change from slab to slab.
  // GRAD_A: H rows are m (out axis): alpha per float4 of the H tile.
  // GRAD_B: H cols are n (out axis): beta float4 per float4 of the H tile.
  float fix_s[TOt::PER];
  float4 fix_v[TOt::PER];
#pragma unroll
  for (int l = 0; l < TOt::PER; ++l) {
    const int idx = tid + l * C::NT;
    if (GRAD_A) {
      fix_s[l] = safe(al, o0 + idx / TOt::C4, M);
    } else {
      const int n = o0 + (idx % TOt::C4) * 4;
      fix_v[l] = make_float4(safe(be, n, N), safe(be, n + 1, N), safe(be, n + 2, N), safe(be, n + 3, N));
    }
  }

  TYt tyl;
  TOt tol, tgl;
  auto load = [&](int q0) __attribute__((always_inline)) {
    tyl.gload(yb, ldy, y0, q0, K, Q, vec_y, tid);
    tol.gload(ob, N, o0, q0, olim, Q, vec_o, tid);
    tgl.gload(gb, N, o0, q0, olim, Q, vec_o, tid);
  };
  if (Q > 0) load(0);
  for (int q0 = 0; q0 < Q; q0 += C::RT) {
    __syncthreads();
    if (GRAD_A) {
      // red axis = n (4 consecutive n per float4): beta float4 shared by Y and H
      {
        const int n = q0 + (tid % TYt::C4) * 4;  // C4 == RT/4 for both tiles; NT % C4 == 0
        const float4 bq = make_float4(safe(be, n, N), safe(be, n + 1, N), safe(be, n + 2, N), safe(be, n + 3, N));
#pragma unroll
        for (int l = 0; l < TYt::PER; ++l) {
          tyl.r[l].x = exp_stage(tyl.r[l].x - bq.x); tyl.r[l].y = exp_stage(tyl.r[l].y - bq.y);
          tyl.r[l].z = exp_stage(tyl.r[l].z - bq.z); tyl.r[l].w = exp_stage(tyl.r[l].w - bq.w);
        }
#pragma unroll
        for (int l = 0; l < TOt::PER; ++l) {
          const float ex = fix_s[l] + bq.x - tol.r[l].x, ey = fix_s[l] + bq.y - tol.r[l].y;
          const float ez = fix_s[l] + bq.z - tol.r[l].z, ew = fix_s[l] + bq.w - tol.r[l].w;
          tol.r[l].x = tgl.r[l].x * exp_stage(ex); tol.r[l].y = tgl.r[l].y * exp_stage(ey);
          tol.r[l].z = tgl.r[l].z * exp_stage(ez); tol.r[l].w = tgl.r[l].w * exp_stage(ew);
        }
      }
    } else {
      // red axis = m (one m per float4 row)
#pragma unroll
      for (int l = 0; l < TYt::PER; ++l) {
        const float s = safe(al, q0 + (tid + l * C::NT) / TYt::C4, M);
        tyl.r[l].x = exp_stage(tyl.r[l].x - s); tyl.r[l].y = exp_stage(tyl.r[l].y - s);
        tyl.r[l].z = exp_stage(tyl.r[l].z - s); tyl.r[l].w = exp_stage(tyl.r[l].w - s);
      }
#pragma unroll
      for (int l = 0; l < TOt::PER; ++l) {
        const float s = safe(al, q0 + (tid + l * C::NT) / TOt::C4, M);
        const float ex = s + fix_v[l].x - tol.r[l].x, ey = s + fix_v[l].y - tol.r[l].y;
        const float ez = s + fix_v[l].z - tol.r[l].z, ew = s + fix_v[l].w - tol.r[l].w;
        tol.r[l].x = tgl.r[l].x * exp_stage(ex); tol.r[l].y = tgl.r[l].y * exp_stage(ey);
        tol.r[l].z = tgl.r[l].z * exp_stage(ez); tol.r[l].w = tgl.r[l].w * exp_stage(ew);
      }
    }
    tyl.sstore(Ys, tid);
    tol.sstore(Hs, tid);
    __syncthreads();
    if (q0 + C::RT < Q) load(q0 + C::RT);
    const int qn = min(C::RT, Q - q0);
    auto step = [&](int qq) __attribute__((always_inline)) {
      if (GRAD_A) {
        float yv[C::TC], hv[C::TR];
        lds_frag<C::TC / 4>(Ys + qq * LDY, tx * 4, C::TX * 4, yv);
        lds_frag<C::TR / 4>(Hs + qq * LDO, ty * C::TR, 4, hv);
#pragma unroll
        for (int i = 0; i < C::TR; ++i)
#pragma unroll
          for (int j = 0; j < C::TC; ++j) acc[i][j] = __builtin_fmaf(hv[i], yv[j], acc[i][j]);
      } else {
        float yv[C::TR], hv[C::TC];
        lds_frag<C::TR / 4>(Ys + qq * LDY, ty * C::TR, 4, yv);
        lds_frag<C::TC / 4>(Hs + qq * LDO, tx * 4, C::TX * 4, hv);
#pragma unroll
        for (int i = 0; i < C::TR; ++i)
#pragma unroll
          for (int j = 0; j < C::TC; ++j) acc[i][j] = __builtin_fmaf(yv[i], hv[j], acc[i][j]);
      }
    };
    if (qn == C::RT) {
#pragma unroll 2
      for (int qq = 0; qq < C::RT; ++qq) step(qq);
    } else {
      for (int qq = 0; qq < qn; ++qq) step(qq);
    }
  }

  // epilogue: grad = exp(x - shift) * acc, x re-read from global memory
  elem_t* gradb = p.grad + (long)batch * R * Cc;
  const float* xshift = GRAD_A ? al : be;  // alpha by row (m) / beta by column (n)
#pragma unroll
  for (int i = 0; i < C::TR; ++i) {
    const int r = r0 + ty * C::TR + i;
    if (r >= R) continue;
    const float rs = GRAD_A ? xshift[r] : 0.f;
#pragma unroll
    for (int q4 = 0; q4 < C::TC / 4; ++q4) {
      const int c = c0 + col_of(4 * q4);
      if (c >= Cc) continue;
      const elem_t* src = xb + (long)r * Cc + c;
      elem_t* dst = gradb + (long)r * Cc + c;
      float xv[4], sv[4];
      const bool full = vec_x && c + 3 < Cc;
      if (full) {
        const float4 v = ld4a(src);
        xv[0] = v.x; xv[1] = v.y; xv[2] = v.z; xv[3] = v.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) xv[e] = (c + e < Cc) ? src[e] : 0.f;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        sv[e] = GRAD_A ? rs : safe(xshift, c + e, Cc);
        xv[e] = exp_comp(xv[e] - sv[e]) * acc[i][4 * q4 + e];
      }
      if (full) {
        st4a(dst, make_float4(xv[0], xv[1], xv[2], xv[3]));
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (c + e < Cc) dst[e] = to_elem<elem_t>(xv[e]);
      }
    }
  }
}

// ----------------------------------------------------------------- dispatch
// `path` (GENBMM_PATH_*): which family of kernels a call may use.  AUTO: whole-item
// kernels for small matrices, the matrix cores where the shape allows, the factored
// vector-ALU kernels otherwise.  EXACT: the online / exp-per-term kernels only (what a
// NULL workspace gives).  VALU: the factored kernels on v_fma_f32, never the matrix cores
// nor the whole-item kernels.  FACTORS: as AUTO, but the matrix-core forward leaves EA, EB and 1/S in
// the workspace and the matrix-core backward reads them instead of forming its operands again from
// a, b, out and the maxima (what AUTO does: the workspace then holds the maxima and flags only).
constexpr int kFixupGrid = 1024;

inline bool valid_path(int path) {
  return path == GENBMM_PATH_AUTO || path == GENBMM_PATH_EXACT || path == GENBMM_PATH_VALU ||
         path == GENBMM_PATH_FACTORS || path == GENBMM_PATH_MFMA32;
}
inline bool auto_path(int path) {
  return path == GENBMM_PATH_AUTO || path == GENBMM_PATH_FACTORS || path == GENBMM_PATH_MFMA32;
}
// MFMA32: as AUTO, but the tiled matrix-core kernels always use the fp32 matrix instruction; under
// AUTO, full-tile shapes run on the bf16 instruction with every factor in three parts (logbmm_split.h).
inline bool split_path(int path) { return path == GENBMM_PATH_AUTO; }
// dynamic LDS beyond 64 KB must be asked for
template <class Kern>
inline void allow_lds(Kern kern, int bytes) {
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

// Layout of the caller's stats buffer: B*(M+N) shifts; one int flag per 32x32
// tile of (M,N) (an upper bound on any forward launch's tile count); a header of
// four ints (which forward filled the buffer, and its tile shape); and, for shapes
// the matrix-core forward can take, its by-products EA (B*M*K), EB (B*K*N) and
// R (B*M*N) on a 16-byte boundary.  Only the forward writes to it.
inline int64_t tiles32(int B, int X, int Y) { return (int64_t)B * ceil_div(X, 32) * ceil_div(Y, 32); }
inline int* fwd_flags_of(const float* stats, int B, int M, int N) {
  return reinterpret_cast<int*>(const_cast<float*>(stats) + (int64_t)B * (M + N));
}
inline int64_t header_offset(int B, int M, int N) {
  const int64_t o = (int64_t)B * (M + N) + tiles32(B, M, N);
  return (o + 3) & ~(int64_t)3;
}
// Small matrices: a whole batch item per workgroup (logbmm_item.h).
inline bool item_shape(int M, int K, int N) {
  return M >= 1 && K >= 1 && N >= 1 && M <= 64 && K <= 64 && N <= 64;
}

// Items of one 128 x 128 tile, each extent large enough for the tile to pay: forward
// and backward form everything they need themselves (logbmm_self.h).
inline bool self_shape(int M, int K, int N) {
  return max(max(M, K), N) <= kSelfMax && min(min(M, K), N) >= 64 && !item_shape(M, K, N);
}

// Shapes whose forward runs on the matrix cores (given alignment and path).
// Extents large enough for 128-wide tiles to pay; ragged edges, odd sizes and
// unaligned rows are handled by the kernels.  (Measured down to a single batch item of 512^3, 16 tiles: the
// matrix-core kernels beat the vector-ALU ones at every tile count.)
inline bool mfma_extents(int out_r, int out_c, int red) {
  return out_r >= 96 && out_c >= 96 && red >= kMS;
}
inline int64_t tiles128(int B, int out_r, int out_c) {
  return (int64_t)B * ceil_div(out_r, 128) * ceil_div(out_c, 128);
}
inline bool fwd_mfma_shape(int B, int M, int K, int N) {
  if (!mfma_extents(M, N, K)) return false;
  const int64_t t128 = tiles128(B, M, N);
  return t128 <= 0x7fffffff;
}
inline LogPrepared prepared_of(const float* stats, int B, int M, int K, int N) {
  float* base = const_cast<float*>(stats) + header_offset(B, M, N);
  LogPrepared w;
  w.hdr = reinterpret_cast<int*>(base);
  w.ea = base + 4;
  w.eb = w.ea + (int64_t)B * M * K;
  w.r = w.eb + (int64_t)B * K * N;
  return w;
}

template <class C>
int launch_fwd_exact(DenseArgs p, int B, int M, int K, int N, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<C>(p, B, M, K, N, grid)) return e;
  hipLaunchKernelGGL((k_log_fwd_exact<C>), grid, dim3(C::NT), 0, s, p);
  return launch_status();
}

template <class CX, int FBM, int FBN>
int launch_fwd_fixup(const DenseArgs& p, const int* flags, int tiles, hipStream_t s) {
  hipLaunchKernelGGL((k_log_fwd_fixup<CX, FBM, FBN>), dim3(min(tiles, kFixupGrid)),
                     dim3(CX::NT), 0, s, p, flags, tiles);
  return launch_status();
}

template <class C, class CX>
int launch_fwd_fast(DenseArgs p, float* stats, int B, int M, int K, int N, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<C>(p, B, M, K, N, grid)) return e;
  int* flags = fwd_flags_of(stats, B, M, N);
  hipLaunchKernelGGL((k_log_fwd_fast<C>), grid, dim3(C::NT), 0, s, p, stats, flags,
                     prepared_of(stats, B, M, K, N).hdr);
  if (int e = launch_status()) return e;
  return launch_fwd_fixup<CX, C::BM, C::BN>(p, flags, (int)grid.x, s);
}

// Matrix-core launches: T is the MTile; the ragged variant of a kernel is used only
// when some extent is not a multiple of its tile / slab.
template <class T>
int launch_fwd_mfma(DenseArgs p, float* stats, int B, int M, int K, int N, bool keep, hipStream_t s) {
  p.M = M; p.K = K; p.N = N;
  p.tiles_m = ceil_div(M, T::TR);
  p.tiles_n = ceil_div(N, T::TC);
  // what the exact fix-up may read and write four aligned elements at a time (the matrix-core
  // kernel itself takes any alignment and ignores these)
  p.vec_a = (K % 4 == 0) && aligned16(p.a);
  p.vec_b = (N % 4 == 0) && aligned16(p.b);
  p.vec_o = (N % 4 == 0) && aligned16(p.out);
  const int total = B * p.tiles_m * p.tiles_n;
  const LogPrepared ws = prepared_of(stats, B, M, K, N);
  int* flags = fwd_flags_of(stats, B, M, N);
  auto go = [&](auto kern) {
    hipLaunchKernelGGL(kern, dim3(total), dim3(T::NT), 0, s, p.a, p.b, p.out, stats, flags, ws.ea,
                       ws.eb, ws.r, ws.hdr, M, K, N, p.tiles_m, p.tiles_n);
  };
  const bool ragged = M % T::TR != 0 || N % T::TC != 0 || K % kMS != 0;
  if (keep) {
    if (ragged) go(k_log_fwd_mfma<T, true, true>);
    else go(k_log_fwd_mfma<T, false, true>);
  } else {
    if (ragged) go(k_log_fwd_mfma<T, true, false>);
    else go(k_log_fwd_mfma<T, false, false>);
  }
  if (int e = launch_status()) return e;
  return launch_fwd_fixup<CfgWide, T::TR, T::TC>(p, flags, total, s);
}

// TF: the forward's tile shape (its flags and the exact fix-up go by it); the sweep
// itself always runs 128 x 128 tiles.
template <class TF>
int launch_sample_sweep_mfma(DenseArgs p, const float* stats, int* flags, int B, int M, int K, int N,
                             hipStream_t s) {
  using T = MTile<128, 128, 2>;
  p.M = M; p.K = K; p.N = N;
  const int tiles_m = ceil_div(M, T::TR), tiles_n = ceil_div(N, T::TC);
  p.tiles_m = ceil_div(M, TF::TR);
  p.tiles_n = ceil_div(N, TF::TC);
  p.vec_a = (K % 4 == 0) && aligned16(p.a);
  p.vec_b = (N % 4 == 0) && aligned16(p.b);
  p.vec_o = (N % 4 == 0) && aligned16(p.out) && aligned16(p.idx);
  const int64_t total = (int64_t)B * tiles_m * tiles_n;
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  const LogPrepared ws = prepared_of(stats, B, M, K, N);
  hipLaunchKernelGGL(k_sample_sweep_split<T>, dim3((unsigned)total), dim3(T::NT), 0, s, ws.ea, ws.eb,
                     p.out, stats, flags, ws.r, p.idx, p.seed, p.offset, M, K, N, tiles_m, tiles_n,
                     TF::TR, TF::TC, p.tiles_m, p.tiles_n, ceil_div(K, kMS) <= 62 ? 63 : 127);
  if (int e = launch_status()) return e;
  const int ftotal = B * p.tiles_m * p.tiles_n;
  hipLaunchKernelGGL((k_sample_fixup<CfgWide, TF::TR, TF::TC>), dim3(min(ftotal, kFixupGrid)),
                     dim3(CfgWide::NT), 0, s, p, flags, ftotal);
  return launch_status();
}

int launch_stats(const elem_t* a, const elem_t* b, float* stats, int B, int M, int K, int N,
                 hipStream_t s) {
  const int row_wgs = ceil_div(M, kStatRows), col_wgs = ceil_div(N, kStatCols);
  const int64_t total = (int64_t)B * (row_wgs + col_wgs);
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  if (total == 0) return GENBMM_OK;
  if (total < 64 && K >= 8192) {  // a handful of workgroups would walk all of K: cut it
    const int kparts = (int)std::min<int64_t>(std::max<int64_t>(256 / (2 * B), 2), K / 2048);
    const int klen = ceil_div(ceil_div(K, kparts), 4) * 4;
    const long count = (long)B * (M + N);
    hipLaunchKernelGGL(k_log_stats_init, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, stats,
                       prepared_of(stats, B, M, K, N).hdr, count);
    hipLaunchKernelGGL(k_log_stats_parts, dim3((unsigned)(2 * B * ceil_div(K, klen))), dim3(256), 0, s, a, b, stats, M, K,
                       N, ceil_div(K, klen), klen);
    return launch_status();
  }
  hipLaunchKernelGGL(k_log_stats, dim3((unsigned)total), dim3(256), 0, s, a, b, stats,
                     prepared_of(stats, B, M, K, N).hdr, M, K, N, row_wgs, col_wgs, (int)((K % 4 == 0) && aligned16(a)),
                     (int)((N % 4 == 0) && aligned16(b)));
  return launch_status();
}

template <class C, bool GRAD_A>
int launch_bwd_exact(LogBwdArgs p, int B, hipStream_t s) {
  const int R = GRAD_A ? p.M : p.K, Cc = GRAD_A ? p.K : p.N;
  p.tiles_r = ceil_div(R, C::BR);
  p.tiles_c = ceil_div(Cc, C::BC);
  const int64_t total = (int64_t)B * p.tiles_r * p.tiles_c;
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  hipLaunchKernelGGL((k_log_bwd_exact<C, GRAD_A>), dim3((unsigned)total), dim3(C::NT), 0, s, p);
  return launch_status();
}

template <class C, class CX, bool GRAD_A>
int launch_bwd_fast(LogBwdArgs p, const float* stats, int B, hipStream_t s) {
  const int R = GRAD_A ? p.M : p.K, Cc = GRAD_A ? p.K : p.N;
  p.tiles_r = ceil_div(R, C::BR);
  p.tiles_c = ceil_div(Cc, C::BC);
  const int64_t total = (int64_t)B * p.tiles_r * p.tiles_c;
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  const int* hdr = prepared_of(stats, B, p.M, p.K, p.N).hdr;
  const int* ff = fwd_flags_of(stats, B, p.M, p.N);
  hipLaunchKernelGGL((k_log_bwd_fast<C, GRAD_A>), dim3((unsigned)total), dim3(C::NT), 0, s, p,
                     stats, hdr, ff);
  if (int e = launch_status()) return e;
  hipLaunchKernelGGL((k_log_bwd_fixup<CX, C::BR, C::BC, GRAD_A>),
                     dim3(min((int)total, kFixupGrid)), dim3(CX::NT), 0, s, p, hdr, ff, 0, (int)total);
  return launch_status();
}

template <class T, bool GRAD_A>
int launch_bwd_mfma(LogBwdArgs p, const float* stats, int B, hipStream_t s, bool lean = false) {
  const int R = GRAD_A ? p.M : p.K, Cc = GRAD_A ? p.K : p.N;
  const int Q = GRAD_A ? p.N : p.M;
  p.tiles_r = ceil_div(R, T::TR);
  p.tiles_c = ceil_div(Cc, T::TC);
  const int total = B * p.tiles_r * p.tiles_c;
  const LogPrepared ws = prepared_of(stats, B, p.M, p.K, p.N);
  const int* ff = fwd_flags_of(stats, B, p.M, p.N);
  auto go = [&](auto kern) {
    hipLaunchKernelGGL(kern, dim3(total), dim3(T::NT), 0, s, p.g, ws.ea, ws.eb, ws.r, ws.hdr, ff,
                       p.grad, p.M, p.K, p.N, p.tiles_r, p.tiles_c);
  };
  auto go_lean = [&](auto kern) {
    hipLaunchKernelGGL(kern, dim3(total), dim3(T::NT), 0, s, p.g, LeanSrc{p.a, p.b, p.out, stats}, ws.hdr, ff, p.grad,
                       p.M, p.K, p.N, p.tiles_r, p.tiles_c);
  };
  const bool ragged = R % T::TR != 0 || Cc % T::TC != 0 || Q % kMS != 0;
  if (lean) {
    if (ragged) go_lean(k_log_bwd_mfma_lean<T, GRAD_A, true>);
    else go_lean(k_log_bwd_mfma_lean<T, GRAD_A, false>);
  } else {
    if (ragged) go(k_log_bwd_mfma<T, GRAD_A, true>);
    else go(k_log_bwd_mfma<T, GRAD_A, false>);
  }
  if (int e = launch_status()) return e;
  hipLaunchKernelGGL((k_log_bwd_fixup<BCfgWide, T::TR, T::TC, GRAD_A>),
                     dim3(min(total, kFixupGrid)), dim3(BCfgWide::NT), 0, s, p, ws.hdr, ff, lean ? 0 : 1, total);
  return launch_status();
}

// grad_a and grad_b of a matrix-core problem in one launch (+ one fix-up launch).
template <class TA, class TB>
int launch_bwd_mfma_both(LogBwdArgs pa, LogBwdArgs pb, const float* stats, int B, hipStream_t s, bool lean = false) {
  const int M = pa.M, K = pa.K, N = pa.N;
  pa.tiles_r = ceil_div(M, TA::TR); pa.tiles_c = ceil_div(K, TA::TC);
  pb.tiles_r = ceil_div(K, TB::TR); pb.tiles_c = ceil_div(N, TB::TC);
  const int64_t ta = (int64_t)B * pa.tiles_r * pa.tiles_c, tb = (int64_t)B * pb.tiles_r * pb.tiles_c;
  if (ta + tb > 0x7fffffffLL) return GENBMM_E_SHAPE;
  const LogPrepared ws = prepared_of(stats, B, M, K, N);
  const int* ff = fwd_flags_of(stats, B, M, N);
  auto go = [&](auto kern) {
    hipLaunchKernelGGL(kern, dim3((unsigned)(ta + tb)), dim3(TA::NT), 0, s, pa.g, ws.ea, ws.eb, ws.r,
                       ws.hdr, ff, pa.grad, pb.grad, M, K, N, (int)ta, pa.tiles_r, pa.tiles_c,
                       pb.tiles_r, pb.tiles_c);
  };
  const bool ragged = M % TA::TR != 0 || K % TA::TC != 0 || N % kMS != 0 || K % TB::TR != 0 ||
                      N % TB::TC != 0 || M % kMS != 0;
  auto go_lean = [&](auto kern) {
    hipLaunchKernelGGL(kern, dim3((unsigned)(ta + tb)), dim3(TA::NT), 0, s, pa.g, LeanSrc{pa.a, pa.b, pa.out, stats},
                       ws.hdr, ff, pa.grad, pb.grad, M, K, N, (int)ta, pa.tiles_r, pa.tiles_c, pb.tiles_r,
                       pb.tiles_c);
  };
  if (lean) {
    if (ragged) go_lean(k_log_bwd_mfma_both_lean<TA, TB, true>);
    else go_lean(k_log_bwd_mfma_both_lean<TA, TB, false>);
  } else {
    if (ragged) go(k_log_bwd_mfma_both<TA, TB, true>);
    else go(k_log_bwd_mfma_both<TA, TB, false>);
  }
  if (int e = launch_status()) return e;
  hipLaunchKernelGGL((k_log_bwd_fixup_both<BCfgWide, TA::TR, TA::TC, TB::TR, TB::TC>),
                     dim3((unsigned)std::min<int64_t>(ta + tb, kFixupGrid)), dim3(BCfgWide::NT), 0,
                     s, pa, pb, ws.hdr, ff, (int)ta, (int)tb, lean ? 0 : 1);
  return launch_status();
}

// The bf16 three-part kernels (logbmm_split.h).  The 256 x 256 tile (one workgroup of sixteen waves
// per compute unit) where both extents split into 256s without more padding than 128-wide tiles
// would add and there are tiles enough to fill the chip; the caller falls back to 256 x 128 /
// 128 x 256.
inline bool pads_to_256(int x) { return ceil_div(x, 256) * 2 == ceil_div(x, 128); }
inline bool split_big_fits(int B, int out_r, int out_c) {
  return pads_to_256(out_r) && pads_to_256(out_c) && (int64_t)B * ceil_div(out_r, 256) * ceil_div(out_c, 256) >= 192;
}
template <class T>
int launch_fwd_split(DenseArgs p, float* stats, int B, int M, int K, int N, bool keep, hipStream_t s) {
  p.M = M; p.K = K; p.N = N;
  p.tiles_m = ceil_div(M, T::TR);
  p.tiles_n = ceil_div(N, T::TC);
  p.vec_a = (K % 4 == 0) && aligned16(p.a);
  p.vec_b = (N % 4 == 0) && aligned16(p.b);
  p.vec_o = (N % 4 == 0) && aligned16(p.out);
  const int64_t total64 = (int64_t)B * p.tiles_m * p.tiles_n;
  if (total64 > 0x7fffffffLL) return GENBMM_E_SHAPE;
  const int total = (int)total64;
  int* flags = fwd_flags_of(stats, B, M, N);
  constexpr int lds = 4 * split_lds_words<SplitT<T::TR, T::NT>, SplitS<T::TC, T::NT>>();
  const LogPrepared ws = prepared_of(stats, B, M, K, N);
  auto go = [&](auto kern) {
    allow_lds(kern, lds);
    hipLaunchKernelGGL(kern, dim3(total), dim3(T::NT), lds, s, p.a, p.b, p.out, stats, flags, ws.ea, ws.eb, ws.r,
                       ws.hdr, M, K, N, p.tiles_m, p.tiles_n, 1);
  };
  const bool ragged = M % T::TR != 0 || N % T::TC != 0 || K % kMS != 0;
  if (keep) {
    if (ragged) go(k_log_fwd_split<T, true, true>);
    else go(k_log_fwd_split<T, false, true>);
  } else {
    if (ragged) go(k_log_fwd_split<T, true, false>);
    else go(k_log_fwd_split<T, false, false>);
  }
  if (int e = launch_status()) return e;
  return launch_fwd_fixup<CfgWide, T::TR, T::TC>(p, flags, total, s);
}
template <class TA, class TB>
int launch_bwd_split_both(LogBwdArgs pa, LogBwdArgs pb, const float* stats, int B, hipStream_t s) {
  const int M = pa.M, K = pa.K, N = pa.N;
  pa.tiles_r = ceil_div(M, TA::TR); pa.tiles_c = ceil_div(K, TA::TC);
  pb.tiles_r = ceil_div(K, TB::TR); pb.tiles_c = ceil_div(N, TB::TC);
  const int64_t ta = (int64_t)B * pa.tiles_r * pa.tiles_c, tb = (int64_t)B * pb.tiles_r * pb.tiles_c;
  if (ta + tb > 0x7fffffffLL) return GENBMM_E_SHAPE;
  const int* hdr = prepared_of(stats, B, M, K, N).hdr;
  const int* ff = fwd_flags_of(stats, B, M, N);
  constexpr int lds = split_bwd_lds_bytes<TA, TB>();
  auto go = [&](auto kern) {
    allow_lds(kern, lds);
    hipLaunchKernelGGL(kern, dim3((unsigned)(ta + tb)), dim3(TA::NT), lds, s, pa.g, LeanSrc{pa.a, pa.b, pa.out, stats},
                       hdr, ff, pa.grad, pb.grad, M, K, N, pa.tiles_r, pa.tiles_c, pb.tiles_r, pb.tiles_c);
  };
  const bool ragged = M % TA::TR != 0 || K % TA::TC != 0 || K % TB::TR != 0 || N % TB::TC != 0 || N % kMS != 0 ||
                      M % kMS != 0;
  if (ragged) go(k_log_bwd_split_both<TA, TB, true>);
  else go(k_log_bwd_split_both<TA, TB, false>);
  if (int e = launch_status()) return e;
  hipLaunchKernelGGL((k_log_bwd_fixup_both<BCfgWide, TA::TR, TA::TC, TB::TR, TB::TC>),
                     dim3((unsigned)std::min<int64_t>(ta + tb, kFixupGrid)), dim3(BCfgWide::NT), 0, s, pa, pb, hdr, ff,
                     (int)ta, (int)tb, 0);
  return launch_status();
}

// Which matrix-core tiling an output of out_r x out_c (reduction over red) gets:
// 2 for the 256-wide tile (when the long side splits into 256s without extra
// padding and there are tiles enough to give every compute unit two workgroups of
// eight waves), 1 for 128x128, 0 for none (path, or extents too small).  `long_cols`:
// the 256 side is the column side of the output.
inline int mfma_kind(int path, int B, int out_r, int out_c, int red, bool long_cols) {
  if (!auto_path(path) || !mfma_extents(out_r, out_c, red)) return 0;
  const int64_t t128 = tiles128(B, out_r, out_c);
  if (t128 > 0x7fffffff) return 0;
  const int L = long_cols ? out_c : out_r;
  if (ceil_div(L, 256) * 2 == ceil_div(L, 128) && t128 >= 512) return 2;
  return 1;
}

using MT128 = MTile<128, 128>;
using MTWide = MTile<128, 256>;  // grad_a (m x k)
using MTTall = MTile<256, 128>;  // forward (m x n; measured 1-2 % ahead of 128x256) and grad_b (k x n)
using MTBig = MTile<256, 256>;   // sixteen waves, one workgroup per compute unit (the bf16 three-part kernels)
using MT128S = MTile<128, 128, 2>;  // the three-part kernels' 128 x 128 tile: a thread stages twice as much, 256 registers

template <bool GRAD_A>
int run_bwd(const LogBwdArgs& p, const float* stats, int path, int B, hipStream_t s) {
  const int R = GRAD_A ? p.M : p.K, Cc = GRAD_A ? p.K : p.N, Q = GRAD_A ? p.N : p.M;
  if ((int64_t)B * R * Cc == 0) return GENBMM_OK;
  auto wgs = [&](int br, int bc) { return (int64_t)B * ceil_div(R, br) * ceil_div(Cc, bc); };
  const bool small = R <= 32 && Cc <= 32;
  if (stats) {
    // the matrix-core kernels run on what the matrix-core forward left behind
    switch (fwd_mfma_shape(B, p.M, p.K, p.N) ? mfma_kind(path, B, R, Cc, Q, GRAD_A) : 0) {
      case 2:
        if constexpr (GRAD_A) return launch_bwd_mfma<MTWide, true>(p, stats, B, s, path != GENBMM_PATH_FACTORS);
        else return launch_bwd_mfma<MTTall, false>(p, stats, B, s, path != GENBMM_PATH_FACTORS);
      case 1: return launch_bwd_mfma<MT128, GRAD_A>(p, stats, B, s, path != GENBMM_PATH_FACTORS);
      default: break;
    }
    if (small) return launch_bwd_fast<BCfgSmall, BCfgSmall, GRAD_A>(p, stats, B, s);
    if (R >= 128 && Cc >= 128 && wgs(128, 128) >= 512)
      return launch_bwd_fast<BCfgBig, BCfgWide, GRAD_A>(p, stats, B, s);
    return launch_bwd_fast<BCfgMid, BCfgMid, GRAD_A>(p, stats, B, s);
  }
  if (small) return launch_bwd_exact<BCfgSmall, GRAD_A>(p, B, s);
  if (R >= 64 && Cc >= 128 && wgs(64, 128) >= 512) return launch_bwd_exact<BCfgWide, GRAD_A>(p, B, s);
  return launch_bwd_exact<BCfgMid, GRAD_A>(p, B, s);
}

template <int G, int TB, bool FULL>
void launch_item_fwd(const elem_t* a, const elem_t* b, elem_t* out, float* stats, int* hdr, int B, int M,
                     int K, int N, hipStream_t s) {
  hipLaunchKernelGGL((k_log_item_fwd<G, TB, FULL>), dim3(B), dim3(G * G), 0, s, a, b, out, stats, hdr, M, K, N);
}

// keep: the workspace is as large as genbmm_logbmm_stats_size says and receives what a
// backward wants beside the maxima; false: header_offset() + 4 floats of it are used.
int launch_self_fwd(DenseArgs p, float* stats, int B, int M, int K, int N, bool split, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<CfgWide>(p, B, M, K, N, grid)) return e;  // what the exact routine reads
  int* hdr = prepared_of(stats, B, M, K, N).hdr;
  const bool full = M == kSelfMax && K == kSelfMax && N == kSelfMax;
  auto go = [&](auto kern) { hipLaunchKernelGGL(kern, dim3(B), dim3(256), 0, s, p, stats, hdr); };
  if (split) {
    if (full) go(k_log_self_fwd<false, true>);
    else go(k_log_self_fwd<true, true>);
  } else {
    if (full) go(k_log_self_fwd<false, false>);
    else go(k_log_self_fwd<true, false>);
  }
  return launch_status();
}

// factors: the caller wants EA, EB and 1/S in the workspace wherever a forward can leave
// them (the sampling sweep), so the kernels that keep no by-products are not used.
// Few output tiles and a long reduction: how many pieces to cut the reduction axis into (1: none).
// At most one round of workgroups over the chip, pieces of at least 32 slabs (512 steps), none empty.
inline int fwd_pieces(int B, int M, int K, int N) {
  const int64_t tiles = tiles128(B, M, N);
  const int slabs = ceil_div(K, kMS);
  if (tiles <= 0 || tiles >= 128 || slabs < 128) return 1;
  const int want = (int)std::min<int64_t>((255 + tiles) / tiles, slabs / 32);
  if (want < 2) return 1;
  return ceil_div(slabs, ceil_div(slabs, want));
}
// The forward in pieces of the reduction axis: 128 x 128 tiles, the pieces' sums in the workspace
// behind the header ([piece][B][M][N]), joined by k_log_fwd_join.
int launch_fwd_pieces(DenseArgs p, float* stats, int B, int M, int K, int N, int pieces, hipStream_t s) {
  using T = MT128S;
  p.M = M; p.K = K; p.N = N;
  p.tiles_m = ceil_div(M, T::TR);
  p.tiles_n = ceil_div(N, T::TC);
  p.vec_a = (K % 4 == 0) && aligned16(p.a);
  p.vec_b = (N % 4 == 0) && aligned16(p.b);
  p.vec_o = (N % 4 == 0) && aligned16(p.out);
  const int total = B * p.tiles_m * p.tiles_n;  // below 128
  int* flags = fwd_flags_of(stats, B, M, N);
  constexpr int lds = 4 * split_lds_words<SplitT<T::TR, T::NT>, SplitS<T::TC, T::NT>>();
  const LogPrepared ws = prepared_of(stats, B, M, K, N);
  float* parts = ws.ea;
  auto kern = k_log_fwd_split<T, true, false, true>;
  allow_lds(kern, lds);
  hipLaunchKernelGGL(kern, dim3(total * pieces), dim3(T::NT), lds, s, p.a, p.b, p.out, stats, flags, nullptr, nullptr,
                     parts, ws.hdr, M, K, N, p.tiles_m, p.tiles_n, pieces);
  if (int e = launch_status()) return e;
  hipLaunchKernelGGL((k_log_fwd_join<T::TR, T::TC>), dim3(total), dim3(256), 0, s, parts, p.out, stats, flags, ws.hdr,
                     B, M, N, p.tiles_m, p.tiles_n, pieces);
  if (int e = launch_status()) return e;
  return launch_fwd_fixup<CfgWide, T::TR, T::TC>(p, flags, total, s);
}
// pieces_ok: the workspace has room for the sums of a forward in pieces (fwd_pieces)
int run_fwd(const elem_t* a, const elem_t* b, elem_t* out, float* stats, int B, int M, int K, int N,
            int path, bool keep, hipStream_t s, bool factors = false, bool pieces_ok = true) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  if (!valid_path(path)) return GENBMM_E_MODE;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn)) return GENBMM_E_NULLPTR;
  if (path != GENBMM_PATH_FACTORS && !factors) keep = false;
  if (stats && B > 0 && item_shape(M, K, N) && auto_path(path)) {  // whole items per workgroup
    int* hdr = prepared_of(stats, B, M, K, N).hdr;
    if (M == 32 && K == 32 && N == 32)  // one wave per item on the matrix cores
      hipLaunchKernelGGL(k_log_item32_fwd, dim3((B + 3) / 4), dim3(256), 0, s, a, b, out, stats, hdr, B);
    else if (M == 64 && K == 64 && N == 64) launch_item_fwd<16, 4, true>(a, b, out, stats, hdr, B, M, K, N, s);
    else if (max(max(M, K), N) <= 32) launch_item_fwd<16, 2, false>(a, b, out, stats, hdr, B, M, K, N, s);
    else launch_item_fwd<16, 4, false>(a, b, out, stats, hdr, B, M, K, N, s);
    return launch_status();
  }
  DenseArgs p{};
  p.a = a; p.b = b; p.out = out; p.idx = nullptr;
  if (stats && B > 0 && self_shape(M, K, N) && auto_path(path) && !factors)
    return launch_self_fwd(p, stats, B, M, K, N, split_path(path), s);
  if (stats) {
    if (int e = launch_stats(a, b, stats, B, M, K, N, s)) return e;
  }
  if (mn == 0) return GENBMM_OK;
  if (stats && split_path(path) && !keep && pieces_ok) {
    const int pieces = fwd_pieces(B, M, K, N);
    if (pieces > 1) return launch_fwd_pieces(p, stats, B, M, K, N, pieces, s);
  }
  if (stats && K > 0 && path != GENBMM_PATH_EXACT) {
    const int64_t big_tiles = (int64_t)B * ceil_div(M, 128) * ceil_div(N, 128);
    switch (fwd_mfma_shape(B, M, K, N) ? mfma_kind(path, B, M, N, K, false) : 0) {
      case 2:
        if (split_path(path)) {
          if (split_big_fits(B, M, N)) return launch_fwd_split<MTBig>(p, stats, B, M, K, N, keep, s);
          return launch_fwd_split<MTTall>(p, stats, B, M, K, N, keep, s);
        }
        return launch_fwd_mfma<MTTall>(p, stats, B, M, K, N, keep, s);
      case 1:
        if (split_path(path)) return launch_fwd_split<MT128S>(p, stats, B, M, K, N, keep, s);
        return launch_fwd_mfma<MT128>(p, stats, B, M, K, N, keep, s);
      default: break;
    }
    if (M <= 32 && N <= 32) return launch_fwd_fast<CfgSmall, CfgSmall>(p, stats, B, M, K, N, s);
    if (M >= 128 && N >= 128 && big_tiles >= 512)
      return launch_fwd_fast<CfgBig, CfgWide>(p, stats, B, M, K, N, s);
    return launch_fwd_fast<CfgMid, CfgMid>(p, stats, B, M, K, N, s);
  }
  switch (pick_shape(B, M, N, false)) {
    case kWide: return launch_fwd_exact<CfgWide>(p, B, M, K, N, s);
    case kMid: return launch_fwd_exact<CfgMid>(p, B, M, K, N, s);
    default: return launch_fwd_exact<CfgSmall>(p, B, M, K, N, s);
  }
}

int run_bwd_both(const elem_t* a, const elem_t* b, const elem_t* out, const elem_t* g,
                 const float* stats, elem_t* grad_a, elem_t* grad_b, int B, int M, int K, int N,
                 int path, hipStream_t s) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  if (!valid_path(path)) return GENBMM_E_MODE;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(g, mn) ||
      (missing(grad_a, mk) && missing(grad_b, kn)))
    return GENBMM_E_NULLPTR;
  LogBwdArgs p{};
  p.a = a; p.b = b; p.out = out; p.g = g;
  p.M = M; p.K = K; p.N = N;
  p.vec_k = (K % 4 == 0) && aligned16(a) && aligned16(grad_a);
  p.vec_n = (N % 4 == 0) && aligned16(b) && aligned16(out) && aligned16(g) && aligned16(grad_b);
  const float* st = (path == GENBMM_PATH_EXACT || mn == 0) ? nullptr : stats;
  if (st && B > 0 && item_shape(M, K, N) && auto_path(path)) {
    if (M == 32 && K == 32 && N == 32)
      hipLaunchKernelGGL(k_log_item32_bwd, dim3((B + 3) / 4), dim3(256), 0, s, a, b, out, g, grad_a, grad_b, B);
    else if (M == 64 && K == 64 && N == 64)
      hipLaunchKernelGGL((k_log_item_bwd<16, 4, true>), dim3(B), dim3(256), 0, s, a, b, out, g, grad_a, grad_b, M, K, N);
    else if (max(max(M, K), N) <= 32)
      hipLaunchKernelGGL((k_log_item_bwd<16, 2>), dim3(B), dim3(256), 0, s, a, b, out, g, grad_a, grad_b, M, K, N);
    else
      hipLaunchKernelGGL((k_log_item_bwd<16, 4>), dim3(B), dim3(256), 0, s, a, b, out, g, grad_a, grad_b, M, K, N);
    return launch_status();
  }
  if (st && B > 0 && self_shape(M, K, N) && auto_path(path)) {
    LogBwdArgs pa = p, pb = p;
    pa.grad = grad_a;
    pb.grad = grad_b;
    const int* hdr = prepared_of(st, B, M, K, N).hdr;
    const dim3 grid((unsigned)ceil_div(B, 8) * 16);
    const bool full = M == kSelfMax && K == kSelfMax && N == kSelfMax;
    auto go = [&](auto kern) { hipLaunchKernelGGL(kern, grid, dim3(256), 0, s, pa, pb, st, hdr, B); };
    if (split_path(path)) {
      if (full) go(k_log_self_bwd<false, true>);
      else go(k_log_self_bwd<true, true>);
    } else {
      if (full) go(k_log_self_bwd<false, false>);
      else go(k_log_self_bwd<true, false>);
    }
    return launch_status();
  }
  if (st && grad_a && grad_b && mk > 0 && kn > 0 && fwd_mfma_shape(B, M, K, N)) {
    const int ka = mfma_kind(path, B, M, K, N, true), kb = mfma_kind(path, B, K, N, M, false);
    if (ka == kb && ka != 0) {
      LogBwdArgs pa = p, pb = p;
      pa.grad = grad_a;
      pb.grad = grad_b;
      const bool lean = path != GENBMM_PATH_FACTORS;
      // (the three-part backward takes any M, and K and N in whole pieces of four - the forward any
      //  sizes -; it addresses a batch item's matrices by 32-bit offsets)
      const bool small_items = (int64_t)M * N < (1ll << 31) && (int64_t)K * N < (1ll << 31) && (int64_t)M * K < (1ll << 31);
      if (lean && split_path(path) && N % 4 == 0 && K % 4 == 0 && small_items) {
        if (ka == 1) return launch_bwd_split_both<MT128S, MT128S>(pa, pb, st, B, s);
        if (split_big_fits(B, M, K) && split_big_fits(B, K, N))
          return launch_bwd_split_both<MTBig, MTBig>(pa, pb, st, B, s);
        return launch_bwd_split_both<MTWide, MTTall>(pa, pb, st, B, s);
      }
      return ka == 2 ? launch_bwd_mfma_both<MTWide, MTTall>(pa, pb, st, B, s, lean)
                     : launch_bwd_mfma_both<MT128, MT128>(pa, pb, st, B, s, lean);
    }
  }
  if (grad_a) {
    p.grad = grad_a;
    if (int e = run_bwd<true>(p, st, path, B, s)) return e;
  }
  if (grad_b) {
    p.grad = grad_b;
    if (int e = run_bwd<false>(p, st, path, B, s)) return e;
  }
  return GENBMM_OK;
}

#if GENBMM_ELEM == 0
// ------------------------------------------------ forward on a workspace of the library's own
// For callers that cannot allocate (code under HIP graph capture, serving loops,
// harnesses that forbid it): the forward's workspace - maxima, per-tile flags, header;
// no by-products for a backward - lives in this array, one copy per GPU for the life
// of the process.  Host code never passes the array's name to a kernel (on the host
// it names a stand-in, not device memory): the device address is looked up once per
// device with that device current and kept in scratch_ptr[].
constexpr size_t kStaticFloats = (size_t)1 << 20;  // 4 MiB
static __device__ __align__(256) float scratch[kStaticFloats];
constexpr int kMaxDevices = 64;
std::mutex scratch_mu;
float* scratch_ptr[kMaxDevices] = {};

int static_workspace(float** ws) {
  int dev = -1;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return GENBMM_E_SHAPE;
  std::lock_guard<std::mutex> lock(scratch_mu);
  if (!scratch_ptr[dev]) {
    float* p = nullptr;
    if (hipError_t e = hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)); e != hipSuccess)
      return (int)e;
    if (!p) return (int)hipErrorInvalidSymbol;
    scratch_ptr[dev] = p;
  }
  *ws = scratch_ptr[dev];
  return GENBMM_OK;
}
#endif

}  // namespace

// The forward's own decision (run_fwd above, path AUTO): factors are written by the
// matrix-core kernels only.
bool log_fwd_writes_factors(const float* stats, int B, int M, int K, int N, LogFactors* f) {
  if (!stats || K <= 0 || (int64_t)B * M * N == 0) return false;
  if (B > 0 && item_shape(M, K, N)) return false;   // whole-item kernels
  if (!fwd_mfma_shape(B, M, K, N)) return false;
  if (mfma_kind(GENBMM_PATH_AUTO, B, M, N, K, false) == 0) return false;
  const LogPrepared ws = prepared_of(stats, B, M, K, N);
  f->ea = ws.ea;
  f->eb = ws.eb;
  f->scratch = ws.r;
  f->valid = ws.hdr;
  return true;
}

int log_fwd_with_factors(const elem_t* a, const elem_t* b, elem_t* out, float* stats, int B, int M, int K,
                         int N, hipStream_t s) {
  return run_fwd(a, b, out, stats, B, M, K, N, GENBMM_PATH_AUTO, true, s, true);
}

bool log_sample_mfma_ok(int K) { return ceil_div(K, kMS) <= kSampleSlabs; }

int log_sample_sweep_mfma(const elem_t* a, const elem_t* b, elem_t* out, int32_t* idx,
                          const float* stats, uint64_t seed, uint64_t offset, int B, int M, int K,
                          int N, hipStream_t s) {
  DenseArgs p{};
  p.a = a; p.b = b; p.out = out; p.idx = idx; p.seed = seed; p.offset = offset;
  if (ceil_div(K, kMS) > kSampleSlabs) return GENBMM_E_SHAPE;  // the caller checks log_sample_mfma_ok
  int* fl = fwd_flags_of(stats, B, M, N);
  // the forward's tile shape: its flags are indexed by it
  switch (mfma_kind(GENBMM_PATH_AUTO, B, M, N, K, false)) {
    case 2:
      if (split_big_fits(B, M, N)) return launch_sample_sweep_mfma<MTBig>(p, stats, fl, B, M, K, N, s);
      return launch_sample_sweep_mfma<MTTall>(p, stats, fl, B, M, K, N, s);
    case 1: return launch_sample_sweep_mfma<MT128>(p, stats, fl, B, M, K, N, s);
    default: return GENBMM_E_SHAPE;
  }
}

// ------------------------------------------------- sampling on a forward in pieces
// One lane per cell, lanes along n.  The cell's target t = u S (u its Philox uniform, S the sum of
// the pieces' sums in the order the join adds them, shrunk by 2^-22 so that it lies inside the
// total) falls into the piece in which the prefix of the pieces' sums passes it; the cell then
// walks that piece's terms exp(a - alpha) exp(b - beta) - the factors whose products the piece's
// sum is - until their prefix passes what was left of t.  The walk's own sum may differ from the
// piece's in the last bits: a target it never reaches names the piece's last term with mass.
// A cell of a tile that the forward flagged (its factored sums are not usable) walks the
// reference's own way: maximum, sum of exponentials, then the decision of
// matmul_cuda_kernel.cu:109-118 on p = exp(a + b - logsumexp), naming the last term that had mass
// when the walk runs out.
__global__ __launch_bounds__(256) void k_sample_cut(const elem_t* __restrict__ a, const elem_t* __restrict__ b,
                                                   const float* __restrict__ stats, const int* __restrict__ flags,
                                                   const float* __restrict__ parts, int32_t* __restrict__ idx,
                                                   uint64_t seed, uint64_t offset, int B, int M, int K, int N,
                                                   int pieces, int slabs_piece, int tiles_m, int tiles_n, long cells) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= cells) return;
  const int n = (int)(e % N);
  const long bm = e / N;
  const int batch = (int)(bm / M), m = (int)(bm - (long)batch * M);
  const elem_t* arow = a + bm * K;
  const elem_t* bcol = b + (long)batch * K * N + n;
  const float u = philox_uniform((uint64_t)e, seed, offset);
  int ind = 0;
  if (flags[((long)batch * tiles_m + m / 128) * tiles_n + n / 128]) {
    float mx = kFloor;
    for (int k = 0; k < K; ++k) mx = __builtin_fmaxf(mx, (float)arow[k] + (float)bcol[(long)k * N]);
    float tot = 0.f;
    for (int k = 0; k < K; ++k) tot += __expf((float)arow[k] + (float)bcol[(long)k * N] - mx);
    const float o = __logf(tot) + mx;
    float acc = 0.f;
    int last = 0;
    bool found = false;
    for (int k = 0; k < K && !found; ++k) {
      const float p = __expf((float)arow[k] + (float)bcol[(long)k * N] - o);
      if (acc <= u && acc + p > u) {  // (<=: a prefix that lands on u exactly must not lose the draw)
        ind = k;
        found = true;
      }
      if (p > 0.f) last = k;
      acc += p;
    }
    if (!found) ind = (acc > 0.f && u >= acc) ? last : 0;  // ran out just below u: the last term with mass
    idx[e] = ind;
    return;
  }
  const float* sp = parts + bm * N + n;  // piece p: sp[p * cells]
  float total = sp[0];
  for (int p = 1; p < pieces; ++p) total += sp[(long)p * cells];
  const float t = u * kSampleShrink * total;
  float before = 0.f;
  int piece = 0;
  for (; piece < pieces - 1; ++piece) {
    const float next = before + sp[(long)piece * cells];
    if (next > t) break;
    before = next;
  }
  const int k0 = piece * slabs_piece * kMS, k1 = min(K, k0 + slabs_piece * kMS);
  const float al = stats[(long)batch * (M + N) + m], be = stats[(long)batch * (M + N) + M + n];
  float rem = t - before;
  int last = k0;
  ind = -1;
  // sixteen terms at a time (their loads in flight together): a group whose sum leaves rem
  // non-negative is passed whole, the group in which rem turns negative is walked term by term
  for (int kc = k0; kc < k1 && ind < 0; kc += 16) {
    float tv[16];
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int k = min(kc + q, k1 - 1);
      tv[q] = fast_exp((float)arow[k] - al) * fast_exp((float)bcol[(long)k * N] - be);
      if (kc + q >= k1) tv[q] = 0.f;
    }
    float sum = 0.f;
#pragma unroll
    for (int q = 0; q < 16; ++q) sum += tv[q];
    const bool whole = rem - sum >= 0.f;
    float r = rem;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      if (tv[q] > 0.f) last = kc + q;
      r -= tv[q];
      if (!whole && ind < 0 && r < 0.f) ind = kc + q;
    }
    rem = whole ? rem - sum : r;
    if (!whole && ind < 0) ind = last;  // the group's sum passed rem, its terms one by one did not: rounding
  }
  idx[e] = ind >= 0 ? ind : last;
}

bool log_sample_cut_ok(const float* stats, int B, int M, int K, int N) {
  return stats != nullptr && (int64_t)B * M * N > 0 && !item_shape(M, K, N) && !self_shape(M, K, N) &&
         fwd_pieces(B, M, K, N) > 1;
}
int64_t log_sample_cut_floats(int B, int M, int K, int N) {
  if ((int64_t)B * M * N == 0 || item_shape(M, K, N) || self_shape(M, K, N)) return 0;
  const int pieces = fwd_pieces(B, M, K, N);
  return pieces > 1 ? (int64_t)pieces * B * M * N : 0;
}
int log_sample_cut(const elem_t* a, const elem_t* b, elem_t* out, int32_t* idx, float* stats, uint64_t seed,
                   uint64_t offset, int B, int M, int K, int N, hipStream_t s) {
  // the forward in pieces: out, the maxima, the flags and every piece's sums
  if (int e = run_fwd(a, b, out, stats, B, M, K, N, GENBMM_PATH_AUTO, false, s, false, true)) return e;
  const int pieces = fwd_pieces(B, M, K, N);
  const int slabs_piece = ceil_div(ceil_div(K, kMS), pieces);
  const long cells = (long)B * M * N;
  if ((cells + 255) / 256 > 0x7fffffffL) return GENBMM_E_SHAPE;
  hipLaunchKernelGGL(k_sample_cut, dim3((unsigned)((cells + 255) / 256)), dim3(256), 0, s, a, b, stats,
                     fwd_flags_of(stats, B, M, N), prepared_of(stats, B, M, K, N).ea, idx, seed, offset, B, M, K, N,
                     pieces, slabs_piece, ceil_div(M, 128), ceil_div(N, 128), cells);
  return launch_status();
}

}  // namespace GENBMM_NS

extern "C" {

#if GENBMM_ELEM == 0
size_t genbmm_logbmm_stats_size_path(int B, int M, int K, int N, int path) {
  using namespace GENBMM_NS;
  if (check_dense_dims(B, M, K, N)) return 0;
  int64_t n = header_offset(B, M, N) + 4;  // maxima, flags and the header
  // the by-products of the matrix-core forward (the one-tile kernels keep the maxima only)
  if (path == GENBMM_PATH_FACTORS && fwd_mfma_shape(B, M, K, N) && !self_shape(M, K, N))
    n += (int64_t)B * ((int64_t)M * K + (int64_t)K * N + (int64_t)M * N);
  // the sums of a forward that cuts a long reduction into pieces
  if (path == GENBMM_PATH_AUTO) {
    const int pieces = fwd_pieces(B, M, K, N);
    if (pieces > 1) n += (int64_t)pieces * B * M * N;
  }
  return (size_t)n;
}

size_t genbmm_logbmm_stats_size(int B, int M, int K, int N) {
  return genbmm_logbmm_stats_size_path(B, M, K, N, GENBMM_PATH_AUTO);
}

int genbmm_logbmm_fwd_pieces(int B, int M, int K, int N) {
  using namespace GENBMM_NS;
  if (check_dense_dims(B, M, K, N) || (int64_t)B * M * N == 0 || item_shape(M, K, N) || self_shape(M, K, N)) return 1;
  return fwd_pieces(B, M, K, N);
}

size_t genbmm_samplebmm_stats_size(int B, int M, int K, int N) {
  using namespace GENBMM_NS;
  if (check_dense_dims(B, M, K, N)) return 0;
  int64_t n = header_offset(B, M, N) + 4;
  // the factors of the matrix-core forward, or the sums of a forward in pieces
  int64_t room = 0;
  if (fwd_mfma_shape(B, M, K, N)) room = (int64_t)B * ((int64_t)M * K + (int64_t)K * N + (int64_t)M * N);
  room = std::max(room, log_sample_cut_floats(B, M, K, N));
  return (size_t)(n + room);
}

size_t genbmm_logbmm_static_limit(void) { return GENBMM_NS::kStaticFloats; }

int genbmm_logbmm_fwd_static(const float* a, const float* b, float* out, int B, int M, int K, int N,
                             void* stream) {
  using namespace GENBMM_NS;
  if (int e = check_dense_dims(B, M, K, N)) return e;
  if ((uint64_t)header_offset(B, M, N) + 4 > kStaticFloats) return GENBMM_E_TOOBIG;
  float* ws = nullptr;
  if (int e = static_workspace(&ws)) return e;
  return run_fwd(a, b, out, ws, B, M, K, N, GENBMM_PATH_AUTO, false, (hipStream_t)stream, false, false);
}
#endif

// The four entry points below exist once per element type: genbmm_logbmm_fwd,
// genbmm_logbmm_fwd_f16, genbmm_logbmm_fwd_bf16, ...
int GENBMM_API(logbmm_fwd)(const GENBMM_NS::abi_t* a, const GENBMM_NS::abi_t* b, GENBMM_NS::abi_t* out,
                           float* stats, int B, int M, int K, int N, void* stream) {
  using namespace GENBMM_NS;
  return run_fwd(el(a), el(b), el(out), stats, B, M, K, N, GENBMM_PATH_AUTO, true, (hipStream_t)stream);
}

int GENBMM_API(logbmm_fwd_path)(const GENBMM_NS::abi_t* a, const GENBMM_NS::abi_t* b,
                                GENBMM_NS::abi_t* out, float* stats, int B, int M, int K, int N,
                                int path, void* stream) {
  using namespace GENBMM_NS;
  return run_fwd(el(a), el(b), el(out), stats, B, M, K, N, path, true, (hipStream_t)stream);
}

int GENBMM_API(logbmm_bwd)(const GENBMM_NS::abi_t* a, const GENBMM_NS::abi_t* b,
                           const GENBMM_NS::abi_t* out, const GENBMM_NS::abi_t* g, const float* stats,
                           GENBMM_NS::abi_t* grad_a, GENBMM_NS::abi_t* grad_b, int B, int M, int K,
                           int N, void* stream) {
  using namespace GENBMM_NS;
  return run_bwd_both(el(a), el(b), el(out), el(g), stats, el(grad_a), el(grad_b), B, M, K, N,
                      GENBMM_PATH_AUTO, (hipStream_t)stream);
}

int GENBMM_API(logbmm_bwd_path)(const GENBMM_NS::abi_t* a, const GENBMM_NS::abi_t* b,
                                const GENBMM_NS::abi_t* out, const GENBMM_NS::abi_t* g,
                                const float* stats, GENBMM_NS::abi_t* grad_a, GENBMM_NS::abi_t* grad_b,
                                int B, int M, int K, int N, int path, void* stream) {
  using namespace GENBMM_NS;
  return run_bwd_both(el(a), el(b), el(out), el(g), stats, el(grad_a), el(grad_b), B, M, K, N, path,
                      (hipStream_t)stream);
}

}  // extern "C"
