// Dense semiring batched matmul, backward and second-order kernels (gfx950).
#include <type_traits>

#include "common.h"

namespace genbmm {
namespace {

// ===================================================== logbmm backward
//
//   w[m,k,n]   = exp(a[m,k] + b[k,n] - out[m,n]) * g[m,n]
//   grad_a[m,k] = sum_n w        grad_b[k,n] = sum_m w
//
// (reference matmul_cuda_backward_kernel_A, matmul_cuda_kernel.cu:159-184,
// where exp(a+b-mx)/exp(out-mx) is the same quantity; the reference obtains
// grad_b by transposing every operand and calling the same kernel again,
// genmul.py:35-41).  The softmax weights are recomputed slab by slab, never
// stored.  One kernel template covers both gradients: the output tile is
// (rows r, cols c) = (m,k) for grad_a or (k,n) for grad_b, and the reduction
// index q is n or m.  X = the operand shaped like the output (kept in
// registers), Y = the other operand, O/G = out and g.
//
//   GRAD_A: Y[q][c] = b[c][q] (out-major), O/G indexed [r][q] (out-major)
//   GRAD_B: Y[q][r] = a[q][r] (red-major), O/G indexed [q][c] (red-major)
template <int BR_, int BC_, int TR_, int TC_, int RT_>
struct BCfg {
  static constexpr int BR = BR_, BC = BC_, TR = TR_, TC = TC_, RT = RT_;
  static constexpr int TX = BC / TC, TY = BR / TR, NT = TX * TY;
  static constexpr int LDR = BR + kPad, LDC = BC + kPad;
};

struct LogBwdArgs {
  const float* a;
  const float* b;
  const float* out;
  const float* g;
  float* grad;
  int M, K, N;
  int tiles_r, tiles_c;
  int vec_k, vec_n;  // float4 access allowed along K-contiguous / N-contiguous rows
};

template <class C, bool GRAD_A>
__global__ __launch_bounds__(C::NT) void k_log_bwd(const LogBwdArgs p) {
  constexpr int BY = GRAD_A ? C::BC : C::BR;   // extent of Y's output axis
  constexpr int BO = GRAD_A ? C::BR : C::BC;   // extent of O/G's output axis
  using TY_t = std::conditional_t<GRAD_A, TileOutMajor<BY, C::RT, C::NT>,
                                  TileRedMajor<BY, C::RT, C::NT>>;
  using TO_t = std::conditional_t<GRAD_A, TileOutMajor<BO, C::RT, C::NT>,
                                  TileRedMajor<BO, C::RT, C::NT>>;
  constexpr int LDY = BY + kPad, LDO = BO + kPad;
  __shared__ __attribute__((aligned(16))) float Ys[C::RT * LDY];
  __shared__ __attribute__((aligned(16))) float Os[C::RT * LDO];
  __shared__ __attribute__((aligned(16))) float Gs[C::RT * LDO];

  const int tid = threadIdx.x, tx = tid % C::TX, ty = tid / C::TX;
  const int M = p.M, K = p.K, N = p.N;
  const int R = GRAD_A ? M : K, Cc = GRAD_A ? K : N, Q = GRAD_A ? N : M;
  const int per = p.tiles_r * p.tiles_c;
  const int batch = blockIdx.x / per;
  const int rem = blockIdx.x - batch * per;
  const int r0 = (rem / p.tiles_c) * C::BR, c0 = (rem % p.tiles_c) * C::BC;

  const float* ab = p.a + (long)batch * M * K;
  const float* bb = p.b + (long)batch * K * N;
  const float* ob = p.out + (long)batch * M * N;
  const float* gb = p.g + (long)batch * M * N;
  const float* xb = GRAD_A ? ab : bb;
  const float* yb = GRAD_A ? bb : ab;
  const long ldy = GRAD_A ? N : K;
  const bool vec_x = GRAD_A ? p.vec_k : p.vec_n;  // X and grad rows are Cc long
  const bool vec_y = GRAD_A ? p.vec_n : p.vec_k;
  const bool vec_o = p.vec_n;
  // output-axis origin / limit of Y and O/G tiles
  const int y0 = GRAD_A ? c0 : r0, ylim = GRAD_A ? K : K;
  const int o0 = GRAD_A ? r0 : c0, olim = GRAD_A ? M : N;

  auto col_of = [&](int j) { return (j >> 2) * (C::TX * 4) + tx * 4 + (j & 3); };

  // X block in registers
  float x[C::TR][C::TC], acc[C::TR][C::TC];
#pragma unroll
  for (int i = 0; i < C::TR; ++i) {
    const int r = r0 + ty * C::TR + i;
#pragma unroll
    for (int q4 = 0; q4 < C::TC / 4; ++q4) {
      const int c = c0 + col_of(4 * q4);
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (r < R && c < Cc) {
        const float* src = xb + (long)r * Cc + c;
        if (vec_x && c + 3 < Cc) {
          v = *reinterpret_cast<const float4*>(src);
        } else {
          v.x = src[0];
          if (c + 1 < Cc) v.y = src[1];
          if (c + 2 < Cc) v.z = src[2];
          if (c + 3 < Cc) v.w = src[3];
        }
      }
      x[i][4 * q4] = v.x; x[i][4 * q4 + 1] = v.y; x[i][4 * q4 + 2] = v.z; x[i][4 * q4 + 3] = v.w;
    }
#pragma unroll
    for (int j = 0; j < C::TC; ++j) acc[i][j] = 0.f;
  }

  TY_t tyl;
  TO_t tol, tgl;
  auto load = [&](int q0) __attribute__((always_inline)) {
    tyl.gload(yb, ldy, y0, q0, ylim, Q, vec_y, tid);
    tol.gload(ob, N, o0, q0, olim, Q, vec_o, tid);
    tgl.gload(gb, N, o0, q0, olim, Q, vec_o, tid);
  };
  if (Q > 0) load(0);
  for (int q0 = 0; q0 < Q; q0 += C::RT) {
    __syncthreads();
#pragma unroll
    for (int l = 0; l < TO_t::PER; ++l) {  // stage -out*log2e
      tol.r[l].x *= -kLog2e; tol.r[l].y *= -kLog2e; tol.r[l].z *= -kLog2e; tol.r[l].w *= -kLog2e;
    }
    tyl.sstore(Ys, tid);
    tol.sstore(Os, tid);
    tgl.sstore(Gs, tid);
    __syncthreads();
    if (q0 + C::RT < Q) load(q0 + C::RT);
    const int qn = min(C::RT, Q - q0);
    auto step = [&](int qq) __attribute__((always_inline)) {
      if (GRAD_A) {
        float yv[C::TC], ov[C::TR], gv[C::TR];
        lds_frag<C::TC / 4>(Ys + qq * LDY, tx * 4, C::TX * 4, yv);
        lds_frag<C::TR / 4>(Os + qq * LDO, ty * C::TR, 4, ov);
        lds_frag<C::TR / 4>(Gs + qq * LDO, ty * C::TR, 4, gv);
#pragma unroll
        for (int i = 0; i < C::TR; ++i)
#pragma unroll
          for (int j = 0; j < C::TC; ++j) {
            const float e = fast_exp2(__builtin_fmaf(x[i][j] + yv[j], kLog2e, ov[i]));
            acc[i][j] = __builtin_fmaf(e, gv[i], acc[i][j]);
          }
      } else {
        float yv[C::TR], ov[C::TC], gv[C::TC];
        lds_frag<C::TR / 4>(Ys + qq * LDY, ty * C::TR, 4, yv);
        lds_frag<C::TC / 4>(Os + qq * LDO, tx * 4, C::TX * 4, ov);
        lds_frag<C::TC / 4>(Gs + qq * LDO, tx * 4, C::TX * 4, gv);
#pragma unroll
        for (int i = 0; i < C::TR; ++i)
#pragma unroll
          for (int j = 0; j < C::TC; ++j) {
            const float e = fast_exp2(__builtin_fmaf(yv[i] + x[i][j], kLog2e, ov[j]));
            acc[i][j] = __builtin_fmaf(e, gv[j], acc[i][j]);
          }
      }
    };
    if (qn == C::RT) {
#pragma unroll 4
      for (int qq = 0; qq < C::RT; ++qq) step(qq);
    } else {
      for (int qq = 0; qq < qn; ++qq) step(qq);
    }
  }

  float* gradb = p.grad + (long)batch * R * Cc;
#pragma unroll
  for (int i = 0; i < C::TR; ++i) {
    const int r = r0 + ty * C::TR + i;
    if (r >= R) continue;
#pragma unroll
    for (int q4 = 0; q4 < C::TC / 4; ++q4) {
      const int c = c0 + col_of(4 * q4);
      float* dst = gradb + (long)r * Cc + c;
      if (vec_x && c + 3 < Cc) {
        *reinterpret_cast<float4*>(dst) =
            make_float4(acc[i][4 * q4], acc[i][4 * q4 + 1], acc[i][4 * q4 + 2], acc[i][4 * q4 + 3]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (c + e < Cc) dst[e] = acc[i][4 * q4 + e];
      }
    }
  }
}

using BCfgWide = BCfg<64, 128, 4, 8, 16>;
using BCfgMid = BCfg<64, 64, 4, 4, 16>;
using BCfgSmall = BCfg<32, 32, 4, 4, 32>;

template <class C, bool GRAD_A>
int launch_log_bwd(LogBwdArgs p, int B, hipStream_t s) {
  const int R = GRAD_A ? p.M : p.K, Cc = GRAD_A ? p.K : p.N;
  if ((int64_t)B * R * Cc == 0) return GENBMM_OK;
  p.tiles_r = ceil_div(R, C::BR);
  p.tiles_c = ceil_div(Cc, C::BC);
  const int64_t total = (int64_t)B * p.tiles_r * p.tiles_c;
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  hipLaunchKernelGGL((k_log_bwd<C, GRAD_A>), dim3((unsigned)total), dim3(C::NT), 0, s, p);
  return launch_status();
}

template <bool GRAD_A>
int run_log_bwd(const LogBwdArgs& p, int B, hipStream_t s) {
  const int R = GRAD_A ? p.M : p.K, Cc = GRAD_A ? p.K : p.N;
  auto wgs = [&](int br, int bc) { return (int64_t)B * ceil_div(R, br) * ceil_div(Cc, bc); };
  if (R <= 32 && Cc <= 32) return launch_log_bwd<BCfgSmall, GRAD_A>(p, B, s);
  if (R >= 64 && Cc >= 128 && wgs(64, 128) >= 512) return launch_log_bwd<BCfgWide, GRAD_A>(p, B, s);
  return launch_log_bwd<BCfgMid, GRAD_A>(p, B, s);
}

// ===================================================== logbmm second order
//
// With p = exp(a+b-out), w = u_a[m,k] + u_b[k,n]  (a missing u counts as 0):
//   t[m,n]      = sum_k p*w                        (gradient w.r.t. g)
//   grad_a[m,k] = sum_n g[m,n]*p*(w - t[m,n])
//   grad_b[k,n] = sum_m g[m,n]*p*(w - t[m,n])
// With u_b = 0 these are the reference's three quartic kernels
// (matmul_cuda_kernel.cu:220-331: inner = sum_k2 (delta*s - s*s2)*u[k2]
// = s*(u[k] - t)), computed in O(M*K*N).  One lane per output element.
struct BB {
  const float* a; const float* b; const float* out; const float* g;
  const float* ua; const float* ub;
  float* ga; float* gb; float* gg;
  int M, K, N;
};

__global__ __launch_bounds__(256) void k_log_bwdbwd_t(const BB p, long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int n = (int)(e % p.N);
  const long bm = e / p.N;  // batch*M + m
  const long batch = bm / p.M;
  const float* arow = p.a + bm * p.K;
  const float* uarow = p.ua ? p.ua + bm * p.K : nullptr;
  const float* bcol = p.b + batch * p.K * p.N + n;
  const float* ubcol = p.ub ? p.ub + batch * p.K * p.N + n : nullptr;
  const float o = p.out[e];
  float t = 0.f;
  for (int k = 0; k < p.K; ++k) {
    const float pr = fast_exp(arow[k] + bcol[(long)k * p.N] - o);
    const float w = (uarow ? uarow[k] : 0.f) + (ubcol ? ubcol[(long)k * p.N] : 0.f);
    t = __builtin_fmaf(pr, w, t);
  }
  p.gg[e] = t;
}

__global__ __launch_bounds__(256) void k_log_bwdbwd_a(const BB p, long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int k = (int)(e % p.K);
  const long bm = e / p.K;
  const long batch = bm / p.M;
  const float av = p.a[e];
  const float uav = p.ua ? p.ua[e] : 0.f;
  const float* brow = p.b + (batch * p.K + k) * p.N;
  const float* ubrow = p.ub ? p.ub + (batch * p.K + k) * p.N : nullptr;
  const float* orow = p.out + bm * p.N;
  const float* grow = p.g + bm * p.N;
  const float* trow = p.gg + bm * p.N;
  float acc = 0.f;
  for (int n = 0; n < p.N; ++n) {
    const float pr = fast_exp(av + brow[n] - orow[n]);
    const float w = uav + (ubrow ? ubrow[n] : 0.f) - trow[n];
    acc = __builtin_fmaf(grow[n] * pr, w, acc);
  }
  p.ga[e] = acc;
}

__global__ __launch_bounds__(256) void k_log_bwdbwd_b(const BB p, long total) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int n = (int)(e % p.N);
  const long bk = e / p.N;  // batch*K + k
  const long batch = bk / p.K;
  const int k = (int)(bk - batch * p.K);
  const float bv = p.b[e];
  const float ubv = p.ub ? p.ub[e] : 0.f;
  const float* acol = p.a + batch * p.M * p.K + k;
  const float* uacol = p.ua ? p.ua + batch * p.M * p.K + k : nullptr;
  const float* ocol = p.out + batch * p.M * p.N + n;
  const float* gcol = p.g + batch * p.M * p.N + n;
  const float* tcol = p.gg + batch * p.M * p.N + n;
  float acc = 0.f;
  for (int m = 0; m < p.M; ++m) {
    const long mn = (long)m * p.N;
    const float pr = fast_exp(acol[(long)m * p.K] + bv - ocol[mn]);
    const float w = (uacol ? uacol[(long)m * p.K] : 0.f) + ubv - tcol[mn];
    acc = __builtin_fmaf(gcol[mn] * pr, w, acc);
  }
  p.gb[e] = acc;
}

// ===================================================== argmax backward
//
// maxbmm / samplebmm:  grad_a[m,k] = sum_n [k == idx[m,n]] g[m,n]
//                      grad_b[k,n] = sum_m [k == idx[m,n]] g[m,n]
// prodmaxbmm: the terms are b[k,n]*g[m,n] and a[m,k]*g[m,n].
// (reference matmul_cuda_kernel.cu:336-456: one thread per gradient cell
// scanning the whole reduction axis, O(M*K*N).)  Here one lane owns one row m
// (resp. column n) and walks it once in ascending n (resp. m), adding each
// term into the cell idx selects, in an LDS-resident accumulator row; the
// additions hitting a given cell therefore happen in the reference's order,
// so the result is bit-identical, in O(M*N) work.  Products are rounded
// before the add (the build uses -ffp-contract=on: no fusion across statements).
constexpr int kKC = 128;  // gradient columns/rows accumulated per pass

template <bool PROD>
__global__ __launch_bounds__(64) void k_argmax_bwd_a(const float* __restrict__ bmat,
                                                    const int32_t* __restrict__ idx,
                                                    const float* __restrict__ g,
                                                    float* __restrict__ grad_a, int M, int K,
                                                    int N, int row_tiles) {
  __shared__ float accs[64 * (kKC + 1)];
  const int lane = threadIdx.x;
  const int batch = blockIdx.x / row_tiles;
  const int m0 = (blockIdx.x - batch * row_tiles) * 64;
  const int m = m0 + lane;
  const bool live = m < M;
  const int32_t* irow = idx + ((long)batch * M + (live ? m : 0)) * N;
  const float* grow = g + ((long)batch * M + (live ? m : 0)) * N;
  const float* bb = PROD ? bmat + (long)batch * K * N : nullptr;
  float* mine = accs + lane * (kKC + 1);
  for (int c0 = 0; c0 < K; c0 += kKC) {
    const int kc = min(kKC, K - c0);
    for (int kk = 0; kk < kKC; ++kk) mine[kk] = 0.f;
    if (live) {
      for (int n = 0; n < N; ++n) {
        const int k = irow[n] - c0;
        if (k >= 0 && k < kc) {
          float v = grow[n];
          if (PROD) v = __fmul_rn(bb[(long)(k + c0) * N + n], v);
          mine[k] = __fadd_rn(mine[k], v);
        }
      }
    }
    __syncthreads();
    const int rows = min(64, M - m0);
    for (int r = 0; r < rows; ++r) {
      float* dst = grad_a + ((long)batch * M + m0 + r) * K + c0;
      for (int kk = lane; kk < kc; kk += 64) dst[kk] = accs[r * (kKC + 1) + kk];
    }
    __syncthreads();
  }
}

template <bool PROD>
__global__ __launch_bounds__(64) void k_argmax_bwd_b(const float* __restrict__ amat,
                                                    const int32_t* __restrict__ idx,
                                                    const float* __restrict__ g,
                                                    float* __restrict__ grad_b, int M, int K,
                                                    int N, int col_tiles) {
  __shared__ float accs[kKC * 64];
  const int lane = threadIdx.x;
  const int batch = blockIdx.x / col_tiles;
  const int n = (blockIdx.x - batch * col_tiles) * 64 + lane;
  if (n >= N) return;  // lanes are independent: no barriers below
  const int32_t* icol = idx + (long)batch * M * N + n;
  const float* gcol = g + (long)batch * M * N + n;
  const float* ab = PROD ? amat + (long)batch * M * K : nullptr;
  for (int c0 = 0; c0 < K; c0 += kKC) {
    const int kc = min(kKC, K - c0);
    for (int kk = 0; kk < kKC; ++kk) accs[kk * 64 + lane] = 0.f;
    for (int m = 0; m < M; ++m) {
      const int k = icol[(long)m * N] - c0;
      if (k >= 0 && k < kc) {
        float v = gcol[(long)m * N];
        if (PROD) v = __fmul_rn(ab[(long)m * K + k + c0], v);
        accs[k * 64 + lane] = __fadd_rn(accs[k * 64 + lane], v);
      }
    }
    for (int kk = 0; kk < kc; ++kk)
      grad_b[((long)batch * K + c0 + kk) * N + n] = accs[kk * 64 + lane];
  }
}

template <bool PROD>
int run_argmax_bwd(const float* a, const float* b, const int32_t* idx, const float* g,
                   float* grad_a, float* grad_b, int B, int M, int K, int N, void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(idx, mn) || missing(g, mn) || missing(grad_a, mk) || missing(grad_b, kn) ||
      (PROD && (missing(a, mk) || missing(b, kn))))
    return GENBMM_E_NULLPTR;
  hipStream_t s = (hipStream_t)stream;
  if ((int64_t)B * M * K > 0) {
    const int row_tiles = ceil_div(M, 64);
    const int64_t total = (int64_t)B * row_tiles;
    if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
    hipLaunchKernelGGL((k_argmax_bwd_a<PROD>), dim3((unsigned)total), dim3(64), 0, s, b, idx, g,
                       grad_a, M, K, N, row_tiles);
    if (int e = launch_status()) return e;
  }
  if ((int64_t)B * K * N > 0) {
    const int col_tiles = ceil_div(N, 64);
    const int64_t total = (int64_t)B * col_tiles;
    if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
    hipLaunchKernelGGL((k_argmax_bwd_b<PROD>), dim3((unsigned)total), dim3(64), 0, s, a, idx, g,
                       grad_b, M, K, N, col_tiles);
    if (int e = launch_status()) return e;
  }
  return GENBMM_OK;
}

}  // namespace
}  // namespace genbmm

extern "C" {

int genbmm_logbmm_bwd(const float* a, const float* b, const float* out, const float* g,
                      float* grad_a, float* grad_b, int B, int M, int K, int N, void* stream) {
  using namespace genbmm;
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(g, mn) ||
      (missing(grad_a, mk) && missing(grad_b, kn)))
    return GENBMM_E_NULLPTR;
  LogBwdArgs p{};
  p.a = a; p.b = b; p.out = out; p.g = g;
  p.M = M; p.K = K; p.N = N;
  p.vec_k = (K % 4 == 0) && aligned16(a) && aligned16(grad_a);
  p.vec_n = (N % 4 == 0) && aligned16(b) && aligned16(out) && aligned16(g) && aligned16(grad_b);
  hipStream_t s = (hipStream_t)stream;
  if (grad_a) {
    p.grad = grad_a;
    if (int e = run_log_bwd<true>(p, B, s)) return e;
  }
  if (grad_b) {
    p.grad = grad_b;
    if (int e = run_log_bwd<false>(p, B, s)) return e;
  }
  return GENBMM_OK;
}

int genbmm_logbmm_bwdbwd(const float* a, const float* b, const float* out, const float* g,
                         const float* u_a, const float* u_b, float* grad_a, float* grad_b,
                         float* grad_g, int B, int M, int K, int N, void* stream) {
  using namespace genbmm;
  if (int e = check_dense_dims(B, M, K, N)) return e;
  {
    const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
    if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(g, mn) ||
        missing(grad_a, mk) || missing(grad_b, kn) || missing(grad_g, mn) ||
        (missing(u_a, mk) && missing(u_b, kn)))
      return GENBMM_E_NULLPTR;
  }
  BB p{a, b, out, g, u_a, u_b, grad_a, grad_b, grad_g, M, K, N};
  hipStream_t s = (hipStream_t)stream;
  auto blocks = [](long total) { return dim3((unsigned)((total + 255) / 256)); };
  const long tmn = (long)B * M * N, tmk = (long)B * M * K, tkn = (long)B * K * N;
  if (tmn > 0) {
    hipLaunchKernelGGL(k_log_bwdbwd_t, blocks(tmn), dim3(256), 0, s, p, tmn);
    if (int e = launch_status()) return e;
  }
  if (tmk > 0) {
    hipLaunchKernelGGL(k_log_bwdbwd_a, blocks(tmk), dim3(256), 0, s, p, tmk);
    if (int e = launch_status()) return e;
  }
  if (tkn > 0) {
    hipLaunchKernelGGL(k_log_bwdbwd_b, blocks(tkn), dim3(256), 0, s, p, tkn);
    if (int e = launch_status()) return e;
  }
  return GENBMM_OK;
}

int genbmm_argmax_bwd(const int32_t* idx, const float* g, float* grad_a, float* grad_b, int B,
                      int M, int K, int N, void* stream) {
  return genbmm::run_argmax_bwd<false>(nullptr, nullptr, idx, g, grad_a, grad_b, B, M, K, N,
                                       stream);
}

int genbmm_prodmax_bwd(const float* a, const float* b, const int32_t* idx, const float* g,
                       float* grad_a, float* grad_b, int B, int M, int K, int N, void* stream) {
  return genbmm::run_argmax_bwd<true>(a, b, idx, g, grad_a, grad_b, B, M, K, N, stream);
}

}  // extern "C"
