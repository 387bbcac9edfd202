// Exact (exp-per-element) logbmm backward tile routine and its configuration.
#pragma once

#include <type_traits>

#include "common.h"

namespace GENBMM_NS {

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
  const elem_t* a;
  const elem_t* b;
  const elem_t* out;
  const elem_t* g;
  elem_t* grad;
  int M, K, N;
  int tiles_r, tiles_c;
  int vec_k, vec_n;  // float4 access allowed along K-contiguous / N-contiguous rows
};

template <class C, bool GRAD_A>
struct LogBwdLds {
  static constexpr int BY = GRAD_A ? C::BC : C::BR;   // extent of Y's output axis
  static constexpr int BO = GRAD_A ? C::BR : C::BC;   // extent of O/G's output axis
  static constexpr int LDY = BY + kPad, LDO = BO + kPad;
  static constexpr int FLOATS = C::RT * (LDY + 2 * LDO);
};

template <class C, bool GRAD_A>
__device__ __forceinline__ void log_bwd_tile(const LogBwdArgs& p, int batch, int r0, int c0,
                                             float* __restrict__ smem) {
  constexpr int BY = GRAD_A ? C::BC : C::BR;   // extent of Y's output axis
  constexpr int BO = GRAD_A ? C::BR : C::BC;   // extent of O/G's output axis
  using TY_t = std::conditional_t<GRAD_A, TileOutMajor<BY, C::RT, C::NT>,
                                  TileRedMajor<BY, C::RT, C::NT>>;
  using TO_t = std::conditional_t<GRAD_A, TileOutMajor<BO, C::RT, C::NT>,
                                  TileRedMajor<BO, C::RT, C::NT>>;
  constexpr int LDY = BY + kPad, LDO = BO + kPad;
  float* Ys = smem;
  float* Os = smem + C::RT * LDY;
  float* Gs = Os + C::RT * LDO;

  const int tid = threadIdx.x, tx = tid % C::TX, ty = tid / C::TX;
  const int M = p.M, K = p.K, N = p.N;
  const int R = GRAD_A ? M : K, Cc = GRAD_A ? K : N, Q = GRAD_A ? N : M;

  const elem_t* ab = p.a + (long)batch * M * K;
  const elem_t* bb = p.b + (long)batch * K * N;
  const elem_t* ob = p.out + (long)batch * M * N;
  const elem_t* gb = p.g + (long)batch * M * N;
  const elem_t* xb = GRAD_A ? ab : bb;
  const elem_t* yb = GRAD_A ? bb : ab;
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
        const elem_t* src = xb + (long)r * Cc + c;
        if (vec_x && c + 3 < Cc) {
          v = ld4a(src);
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

  elem_t* gradb = p.grad + (long)batch * R * Cc;
#pragma unroll
  for (int i = 0; i < C::TR; ++i) {
    const int r = r0 + ty * C::TR + i;
    if (r >= R) continue;
#pragma unroll
    for (int q4 = 0; q4 < C::TC / 4; ++q4) {
      const int c = c0 + col_of(4 * q4);
      elem_t* dst = gradb + (long)r * Cc + c;
      if (vec_x && c + 3 < Cc) {
        st4a(dst, make_float4(acc[i][4 * q4], acc[i][4 * q4 + 1], acc[i][4 * q4 + 2], acc[i][4 * q4 + 3]));
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (c + e < Cc) dst[e] = to_elem<elem_t>(acc[i][4 * q4 + e]);
      }
    }
  }
}

using BCfgBig = BCfg<128, 128, 8, 8, 16>;
using BCfgWide = BCfg<64, 128, 4, 8, 16>;
using BCfgMid = BCfg<64, 64, 4, 4, 16>;
using BCfgSmall = BCfg<32, 32, 4, 4, 32>;

}  // namespace GENBMM_NS
