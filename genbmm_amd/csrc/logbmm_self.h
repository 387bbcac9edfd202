// logbmm for batch items whose three extents are all at most 128: the whole
// item is one 128 x 128 tile, so a workgroup can do everything the larger
// problems need separate launches and a large workspace for.
//
// Forward (one workgroup of four waves per item): every thread requests its
// share of a and b for ALL reduction slabs at once (32 16-byte loads in flight
// per lane, the item read from memory exactly once), the row maxima of a and
// the column maxima of b are reduced from those registers (no pass of their
// own), the exponentials are taken while the slabs are staged into LDS, the
// contraction runs on v_mfma_f32_32x32x2_f32, and a tile that fails the
// factoring guard is redone on the spot by the online log-sum-exp routine
// (no fix-up launch, no flags).  The workspace receives the maxima only.
//
// Backward (two workgroups per item, one per gradient, neighbours on one XCD so
// that the second read of the operands comes from that XCD's L2): the factors
// are formed again from a, b, out and the maxima while staging -
// EA = exp(a - alpha), EB = exp(b - beta), H = g * exp(alpha + beta - out) -
// instead of being read back: 4 matrices in, 2 out, nothing else moves.  The
// guard is evaluated on out - alpha - beta, so it does not depend on which
// kernel produced `out`; a failing item is redone by the exact exp(a+b-out) routine.
#pragma once

#include "dense_tiles.h"
#include "log_bwd_tile.h"
#include "logbmm_mfma.h"
#include "logbmm_split.h"
#include "logbmm_ws.h"

namespace GENBMM_NS {

constexpr int kSelfMax = 128;               // largest extent these kernels take
constexpr int kSelfSlabs = kSelfMax / kMS;  // reduction slabs at that extent
using SelfTile = MTile<kSelfMax, kSelfMax, 2>;
// SPLIT kernels: the products on the bf16 matrix instruction, every staged factor in three bf16
// parts (logbmm_split.h); the staged form takes more LDS than the fp32 one, which sets the size.
using SelfSplitT = SplitT<kSelfMax, SelfTile::NT>;
using SelfSplitS = SplitS<kSelfMax, SelfTile::NT>;
constexpr int kSelfLds = 4 * SelfSplitS::BUF;  // two buffers of two operands, each the size of the larger form
static_assert(kSelfLds >= 2 * kMS * (SelfTile::LDR + SelfTile::LDC) && SelfSplitT::BUF <= SelfSplitS::BUF, "");
// Pieces of an operand stored [reduction][line]: rows red(tid, l), l = 0, 1, of a slab, four
// lines from quad * 4.  The bf16 form wants a thread's two rows to be neighbours (a pair shares
// a word); the fp32 form has them eight apart (StageS).
template <bool SPLIT>
struct SelfS {
  static __device__ __forceinline__ int red(int tid, int l) { return SPLIT ? 2 * (tid >> 5) + l : (tid >> 5) + 8 * l; }
  static __device__ __forceinline__ int quad(int tid) { return tid & 31; }
};
// the two LDS buffers of a split operand pair, rows operand first (sizes of the larger form)
__device__ __forceinline__ unsigned* self_split_rows(float* smem, int buf) {
  return reinterpret_cast<unsigned*>(smem) + buf * SelfSplitS::BUF;
}
__device__ __forceinline__ unsigned* self_split_cols(float* smem, int buf) {
  return reinterpret_cast<unsigned*>(smem) + (2 + buf) * SelfSplitS::BUF;
}
static_assert(kSelfLds >= CfgWide::KT * (CfgWide::LDA + CfgWide::LDB), "exact forward routine fits");
static_assert(kSelfLds >= LogBwdLds<BCfgWide, true>::FLOATS && kSelfLds >= LogBwdLds<BCfgWide, false>::FLOATS,
              "exact backward routine fits");
// S >= 2^-40 written for d = alpha + beta - out = -log S
constexpr float kSelfGuardD = kMfmaGuardBits * kLn2;

__device__ __forceinline__ float max4(float4 v) { return fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w)); }
__device__ __forceinline__ float4 fmax4(float4 x, float4 y) {
  return make_float4(fmaxf(x.x, y.x), fmaxf(x.y, y.y), fmaxf(x.z, y.z), fmaxf(x.w, y.w));
}
template <int I, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < E) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, E>(f);
  }
}
// The shifts of an item, one per thread (`row`: a row's maximum, else a column's; `here`: the
// thread has one): may the item be factored?  Every shift finite and not below the reference's
// floor, and - the reference keeps its running maximum at the floor or above, and its terms
// vanish from about 100 below it - no row at the floor (an operand row padded with -1e9) together
// with a column whose shift is below -30, nor the other way round.  Every thread of the
// workgroup calls this (it synchronizes); the answer is uniform.
__device__ __forceinline__ int self_shifts_bad(bool here, bool row, float sh) {
  int bad = 0, low = 0, neg = 0;  // bit 0: of a row, bit 1: of a column
  if (here) {
    bad = !((sh >= kFloor) && (sh < INFINITY));
    if (sh <= 0.45f * kFloor) low = row ? 1 : 2;
    if (sh < -30.f) neg = row ? 1 : 2;
  }
  const int row_low = __syncthreads_or(low & 1), col_low = __syncthreads_or(low & 2);
  if (row_low | col_low) {  // uniform, and rare
    const int row_neg = __syncthreads_or(neg & 1), col_neg = __syncthreads_or(neg & 2);
    if ((row_low && col_neg) || (col_low && row_neg)) bad = 1;
  }
  return __syncthreads_or(bad);
}

// ----------------------------------------------------------------- forward
// An item that fails the guard: the online routine, two 64 x 128 tiles.
__device__ __forceinline__ void self_fwd_exact(const DenseArgs& p, int batch, float* smem) {
  for (int h = 0; h < kSelfMax / CfgWide::BM; ++h)
    if (h * CfgWide::BM < p.M) {
      log_fwd_tile<CfgWide, false>(p, batch, h * CfgWide::BM, 0, smem, smem + CfgWide::KT * CfgWide::LDA);
      __syncthreads();
    }
}

template <bool RAGGED, bool SPLIT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void k_log_self_fwd(const DenseArgs p, float* __restrict__ stats, int* __restrict__ hdr) {
  using T = SelfTile;
  constexpr int NT = T::NT, LD = T::LDR;
  static_assert(NT == 256 && T::LDR == T::LDC && CfgWide::NT == 256, "");
  using SA = StageT<kSelfMax, NT, LD>;
  using SB = StageS<kSelfMax, NT, LD>;
  using SBr = SelfS<SPLIT>;
  static_assert(SA::PER == 2 && SB::PER == 2 && SelfSplitT::PER == 2, "");
  __shared__ __attribute__((aligned(16))) float smem[kSelfLds];
  __shared__ __attribute__((aligned(16))) float s_al[kSelfMax], s_be[kSelfMax], s_part[4][kSelfMax];
  float(*As)[kMS * LD] = reinterpret_cast<float(*)[kMS * LD]>(smem);
  float(*Bs)[kMS * LD] = reinterpret_cast<float(*)[kMS * LD]>(smem + 2 * kMS * LD);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
  const int batch = blockIdx.x;
  const int M = p.M, K = p.K, N = p.N;
  const elem_t* ab = p.a + (long)batch * M * K;
  const elem_t* bb = p.b + (long)batch * K * N;
  float* st = stats + (long)batch * (M + N);
  const int slabs = RAGGED ? (K + kMS - 1) / kMS : kSelfSlabs;
  const float4 ninf = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
  if (batch == 0 && tid == 0) {
    hdr[1] = T::TR;
    hdr[2] = T::TC;
    hdr[0] = kWsSelf;
  }

  // the whole item, requested at once
  const int aq = SA::quad(tid) * 4;                     // a pieces: four k from 16 s + aq
  const int bcol = SB::quad(tid) * 4;                   // b pieces: four n from bcol
  const int cb = RAGGED ? clamp4(N - bcol) : 4;
  float4 ra[kSelfSlabs][2], rb[kSelfSlabs][2];
  // (uniform base + 32-bit lane offset + constant: two registers of addressing per operand)
  unsigned oa[2], obb[2];
#pragma unroll
  for (int l = 0; l < 2; ++l) {
    oa[l] = (unsigned)(SA::line(tid, l) * K + aq);
    obb[l] = (unsigned)(SBr::red(tid, l) * N + bcol);
  }
#pragma unroll
  for (int s = 0; s < kSelfSlabs; ++s)
    if (!RAGGED || s < slabs) {
      const elem_t* bs = bb + (size_t)(kMS * s) * N;  // uniform
#pragma unroll
      for (int l = 0; l < 2; ++l) {
        const int m = SA::line(tid, l), k = kMS * s + SBr::red(tid, l);
        if (!RAGGED) {
          ra[s][l] = ld4(ab + oa[l] + kMS * s);
          rb[s][l] = ld4(bs + obb[l]);
        } else {
          ra[s][l] = m < M ? ld4m(ab + oa[l] + kMS * s, K - (kMS * s + aq), -INFINITY) : ninf;
          rb[s][l] = k < K ? ld4m(bs + obb[l], cb, -INFINITY) : ninf;
        }
      }
    }

  // alpha: the four lanes of a line hold its row between them
  float al[2];
#pragma unroll
  for (int l = 0; l < 2; ++l) {
    float m = -INFINITY;
#pragma unroll
    for (int s = 0; s < kSelfSlabs; ++s)
      if (!RAGGED || s < slabs) m = fmaxf(m, max4(ra[s][l]));
    m = fmaxf(m, __shfl_xor(m, 1, 64));
    m = fmaxf(m, __shfl_xor(m, 2, 64));
    const int line = SA::line(tid, l);
    const bool here = !RAGGED || line < M;
    al[l] = here ? m : INFINITY;  // lines beyond the matrix: exp -> 0
    if ((tid & 3) == 0) {
      s_al[line] = al[l];
      if (here) st[line] = m;
    }
  }
  // beta: a column's terms sit in the same lane position of all eight half-waves
  float4 be = ninf;
#pragma unroll
  for (int s = 0; s < kSelfSlabs; ++s)
    if (!RAGGED || s < slabs) be = fmax4(be, fmax4(rb[s][0], rb[s][1]));
  be.x = fmaxf(be.x, __shfl_xor(be.x, 32, 64));
  be.y = fmaxf(be.y, __shfl_xor(be.y, 32, 64));
  be.z = fmaxf(be.z, __shfl_xor(be.z, 32, 64));
  be.w = fmaxf(be.w, __shfl_xor(be.w, 32, 64));
  if (lane < 32) *reinterpret_cast<float4*>(&s_part[wave][bcol]) = be;
  __syncthreads();
  be = fmax4(fmax4(*reinterpret_cast<const float4*>(&s_part[0][bcol]),
                   *reinterpret_cast<const float4*>(&s_part[1][bcol])),
             fmax4(*reinterpret_cast<const float4*>(&s_part[2][bcol]),
                   *reinterpret_cast<const float4*>(&s_part[3][bcol])));
  if (tid < 32) {
    if (RAGGED) st4m(st + M + (cb > 0 ? bcol : 0), cb, be);
    else st4(st + M + bcol, be);
  }
  if (RAGGED) {  // columns beyond the matrix: exp -> 0
    if (cb < 1) be.x = INFINITY;
    if (cb < 2) be.y = INFINITY;
    if (cb < 3) be.z = INFINITY;
    if (cb < 4) be.w = INFINITY;
  }
  if (tid < 32) *reinterpret_cast<float4*>(&s_be[bcol]) = be;

  floatx16 acc[2][2];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[x >> 1][x & 1][i] = 0.f;

#pragma unroll
  for (int s = 0; s <= kSelfSlabs; ++s) {
    // slab s is staged while slab s-1 is multiplied
    if (s < kSelfSlabs && (!RAGGED || s < slabs)) {
      if constexpr (SPLIT) {
#pragma unroll
        for (int l = 0; l < 2; ++l) SelfSplitT::put(self_split_rows(smem, s & 1), tid, l, exp4(ra[s][l], al[l]));
        SelfSplitS::put(self_split_cols(smem, s & 1), tid, exp4(rb[s][0], be), exp4(rb[s][1], be));
      } else {
#pragma unroll
        for (int l = 0; l < 2; ++l) {
          SA::put(As[s & 1], tid, l, exp4(ra[s][l], al[l]));
          SB::put(Bs[s & 1], tid, l, exp4(rb[s][l], be));
        }
      }
    }
    if (s > 0 && (!RAGGED || s <= slabs)) {
      if constexpr (SPLIT)
        split_slab<SelfSplitT, SelfSplitS>(self_split_rows(smem, (s - 1) & 1), self_split_cols(smem, (s - 1) & 1), wm0, wn0,
                                           wave, lane, acc);
      else
        mfma_slab<LD, LD>(As[(s - 1) & 1], Bs[(s - 1) & 1], wm0, wn0, lane, acc);
    }
    __syncthreads();
  }

  // guard: S >= 2^-40 and finite, every shift finite and far above the -1e9 floor
  const float thr = fast_exp2(-kMfmaGuardBits);
  int bad = 0;
  {
    const int rlim = M - wm0 - mfma_row_l(lane);
    const int clim = N - wn0 - (lane & 31);
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float s = acc[x >> 1][x & 1][i];
        const bool here = !RAGGED || ((x >> 1) * 32 + mfma_row_u(i) < rlim && (x & 1) * 32 < clim);
        if (here && !((s >= thr) && (s < INFINITY))) bad = 1;
      }
  }
  {
    const bool row = tid < kSelfMax;
    const int t = row ? tid : tid - kSelfMax;
    const bool here = !RAGGED || t < (row ? M : N);
    bad |= self_shifts_bad(here, row, here ? (row ? s_al[t] : s_be[t]) : 0.f);
  }
  bad = __builtin_amdgcn_readfirstlane(__syncthreads_or(bad));
  if (bad) {
    self_fwd_exact(p, batch, smem);
    return;
  }

  // out = log S + alpha + beta, written row-wise
  const int lr = lane >> 4, lc = (lane & 15) * 4;
  const int cc = RAGGED ? clamp4(N - (wn0 + lc)) : 4;
  const bool cok = cc > 0;
  const float4 be4 = *reinterpret_cast<const float4*>(&s_be[wn0 + lc]);
  const float* alw = s_al + wm0 + lr;
  elem_t* ob = p.out + ((long)batch * M + wm0 + lr) * N + wn0 + lc;
  const int rows_left = M - wm0 - lr;
  acc_rows(acc, smem + wave * kStripFloats, lane, [](int) {},
           [&](int q, int t, float4 sv) __attribute__((always_inline)) {
             const int ru = 16 * q + 4 * t;
             if (RAGGED && !(cok && ru < rows_left)) return;
             const float alr = alw[ru];
             const float4 ov = make_float4(__builtin_fmaf(fast_log2(sv.x), kLn2, alr + be4.x),
                                           __builtin_fmaf(fast_log2(sv.y), kLn2, alr + be4.y),
                                           __builtin_fmaf(fast_log2(sv.z), kLn2, alr + be4.z),
                                           __builtin_fmaf(fast_log2(sv.w), kLn2, alr + be4.w));
             if (RAGGED) st4m(ob + (long)ru * N, cc, ov);
             else st4(ob + (long)ru * N, ov);
           });
}

// ---------------------------------------------------------------- backward
// An item that fails the guard: the exact routine, two 64 x 128 tiles.
template <bool GRAD_A>
__device__ __forceinline__ void self_bwd_exact(const LogBwdArgs& p, int batch, float* smem) {
  const int R = GRAD_A ? p.M : p.K;
  for (int h = 0; h < kSelfMax / BCfgWide::BR; ++h)
    if (h * BCfgWide::BR < R) {
      log_bwd_tile<BCfgWide, GRAD_A>(p, batch, h * BCfgWide::BR, 0, smem);
      __syncthreads();
    }
}

// H piece from g, out and the shifts; cells beyond the matrix (cnt) give 0 and do not
// take part in the guard.
template <bool RAGGED>
__device__ __forceinline__ float4 self_h(float4 g, float4 o, float4 sh, int cnt, int& bad) {
  const float dx = sh.x - o.x, dy = sh.y - o.y, dz = sh.z - o.z, dw = sh.w - o.w;
  auto ok = [](float d) { return (d < kSelfGuardD) && (d > -128.f); };
  float4 h = make_float4(g.x * exp_st(dx), g.y * exp_st(dy), g.z * exp_st(dz), g.w * exp_st(dw));
  if (!RAGGED) {
    if (!(ok(dx) && ok(dy) && ok(dz) && ok(dw))) bad = 1;
  } else {
    if ((cnt > 0 && !ok(dx)) || (cnt > 1 && !ok(dy)) || (cnt > 2 && !ok(dz)) || (cnt > 3 && !ok(dw))) bad = 1;
    if (cnt < 1) h.x = 0.f;
    if (cnt < 2) h.y = 0.f;
    if (cnt < 3) h.z = 0.f;
    if (cnt < 4) h.w = 0.f;
  }
  // H is formed here, not after the branch on the guard (where the compiler would move it,
  // keeping g and the exponents alive in its place)
  asm volatile("" : "+v"(h.x), "+v"(h.y), "+v"(h.z), "+v"(h.w));
  return h;
}

template <bool GRAD_A, bool RAGGED, bool SPLIT>
__device__ __forceinline__ void log_self_bwd_tile(float* __restrict__ smem, float* __restrict__ s_al,
                                                  float* __restrict__ s_be, const LogBwdArgs& p,
                                                  const float* __restrict__ stats,
                                                  const int* __restrict__ hdr, int batch) {
  using T = SelfTile;
  constexpr int NT = T::NT, LD = T::LDR;
  using ST = StageT<kSelfMax, NT, LD>;  // sources [out][red]: both operands of grad_a
  using SP = StageS<kSelfMax, NT, LD>;  // sources [red][out]: both operands of grad_b ...
  using SS = SelfS<SPLIT>;              // ... and which pieces a thread holds of them
  float(*Rs)[kMS * LD] = reinterpret_cast<float(*)[kMS * LD]>(smem);
  float(*Cs)[kMS * LD] = reinterpret_cast<float(*)[kMS * LD]>(smem + 2 * kMS * LD);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr0 = (wave >> 1) * 64, wc0 = (wave & 1) * 64;
  const int M = p.M, K = p.K, N = p.N;
  const int Q = GRAD_A ? N : M, R = GRAD_A ? M : K, Cc = GRAD_A ? K : N;
  const elem_t* ab = p.a + (long)batch * M * K;
  const elem_t* bb = p.b + (long)batch * K * N;
  const elem_t* ob = p.out + (long)batch * M * N;
  const elem_t* gb = p.g + (long)batch * M * N;
  const float* st = stats + (long)batch * (M + N);
  const int slabs = RAGGED ? (Q + kMS - 1) / kMS : kSelfSlabs;
  const float4 ninf = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);

  // the shifts the forward left (any forward that writes them will do)
  const int tag = hdr[0];
  int bad = !(tag == kWsSelf || tag == kWsMfma || tag == kWsFast);
  float my_shift;
  {
    const bool row = tid < kSelfMax;
    const int t = row ? tid : tid - kSelfMax;
    const bool here = !RAGGED || t < (row ? M : N);
    my_shift = here ? st[row ? t : M + t] : 0.f;
    (row ? s_al : s_be)[t] = my_shift;
  }

  // What this tile stages: rg/ro = g and out, ry = the other operand.  g and out are requested at
  // once (32 16-byte loads in flight per lane); the other operand's pieces follow two slabs ahead
  // of the staging, into registers that `out` pieces have left.
  float4 rg[kSelfSlabs][2], ro[kSelfSlabs][2], ry[kSelfSlabs][2];
  const int tq = ST::quad(tid) * 4;   // grad_a: four reduction steps n from 16 s + tq
  const int sc = SS::quad(tid) * 4;   // grad_b: four output columns from sc (k of EA, n of H)
  const int ck = RAGGED ? clamp4(K - sc) : 4, cn = RAGGED ? clamp4(N - sc) : 4;
  // (uniform base + 32-bit lane offset + constant: two registers of addressing per operand)
  unsigned on[2], oy[2];
#pragma unroll
  for (int l = 0; l < 2; ++l) {
    on[l] = GRAD_A ? (unsigned)(ST::line(tid, l) * N + tq) : (unsigned)(SS::red(tid, l) * N + sc);
    oy[l] = GRAD_A ? on[l] : (unsigned)(SS::red(tid, l) * K + sc);
  }
  // grad_a walks along the rows (a constant per slab), grad_b down the rows (uniform pointers)
  auto load_h = [&](auto sc_) __attribute__((always_inline)) {
    constexpr int s = decltype(sc_)::value;
    if (RAGGED && s >= slabs) return;
    const size_t dn = GRAD_A ? (size_t)(kMS * s) : (size_t)(kMS * s) * N;
    const elem_t* gs = gb + dn;
    const elem_t* os = ob + dn;
#pragma unroll
    for (int l = 0; l < 2; ++l) {
      if (!RAGGED) {
        rg[s][l] = ld4(gs + on[l]);
        ro[s][l] = ld4(os + on[l]);
      } else {
        const bool rowin = (GRAD_A ? ST::line(tid, l) : kMS * s + SS::red(tid, l)) < M;
        const int cnt = GRAD_A ? N - (kMS * s + tq) : cn;
        rg[s][l] = rowin ? ld4m(gs + on[l], cnt, 0.f) : zero4;
        ro[s][l] = rowin ? ld4m(os + on[l], cnt, 0.f) : zero4;
      }
    }
  };
  auto load_y = [&](auto sc_) __attribute__((always_inline)) {
    constexpr int s = decltype(sc_)::value;
    if (RAGGED && s >= slabs) return;
    const elem_t* ys = (GRAD_A ? bb : ab) + (GRAD_A ? (size_t)(kMS * s) : (size_t)(kMS * s) * K);
#pragma unroll
    for (int l = 0; l < 2; ++l) {
      if (!RAGGED) ry[s][l] = ld4(ys + oy[l]);
      else if constexpr (GRAD_A)  // EB[k][n]: line k, four n
        ry[s][l] = ST::line(tid, l) < K ? ld4m(ys + oy[l], N - (kMS * s + tq), -INFINITY) : ninf;
      else                        // EA[m][k]: row m, four k
        ry[s][l] = kMS * s + SS::red(tid, l) < M ? ld4m(ys + oy[l], ck, -INFINITY) : ninf;
    }
  };
  // H (into rg) with the guard on every cell of out, and the other factor (into ry)
  auto make_h = [&](auto sc_) __attribute__((always_inline)) {
    constexpr int s = decltype(sc_)::value;
    if (RAGGED && s >= slabs) return;
#pragma unroll
    for (int l = 0; l < 2; ++l) {
      const int row = GRAD_A ? ST::line(tid, l) : kMS * s + SS::red(tid, l);  // m
      const int col = GRAD_A ? kMS * s + tq : sc;                             // n
      const float4 bq = *reinterpret_cast<const float4*>(&s_be[col]);
      const float alm = s_al[row];
      const int cnt = RAGGED ? (row < M ? clamp4(N - col) : 0) : 4;
      rg[s][l] = self_h<RAGGED>(rg[s][l], ro[s][l],
                                make_float4(alm + bq.x, alm + bq.y, alm + bq.z, alm + bq.w), cnt, bad);
    }
  };
  auto make_y = [&](auto sc_) __attribute__((always_inline)) {
    constexpr int s = decltype(sc_)::value;
    if (RAGGED && s >= slabs) return;
#pragma unroll
    for (int l = 0; l < 2; ++l) {
      if constexpr (GRAD_A) ry[s][l] = exp4(ry[s][l], *reinterpret_cast<const float4*>(&s_be[kMS * s + tq]));
      else ry[s][l] = exp4(ry[s][l], s_al[kMS * s + SS::red(tid, l)]);
    }
  };
  constexpr int kAhead = 4;  // slabs the other operand's loads run ahead of the staging
  static_for<0, kAhead>(load_y);  // first: the memory counter retires loads in issue order
  __builtin_amdgcn_sched_barrier(0);
  static_for<0, kSelfSlabs>(load_h);
  __builtin_amdgcn_sched_barrier(0);
  __syncthreads();  // s_al, s_be
  {  // (asked here, behind the loads: it waits for the shifts)
    const bool row = tid < kSelfMax;
    const int t = row ? tid : tid - kSelfMax;
    bad |= self_shifts_bad(!RAGGED || t < (row ? M : N), row, my_shift);
  }

  floatx16 acc[2][2];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[x >> 1][x & 1][i] = 0.f;

  auto multiply = [&](int buf) __attribute__((always_inline)) {
    if constexpr (!SPLIT) mfma_slab<LD, LD>(Rs[buf], Cs[buf], wr0, wc0, lane, acc);
    else if constexpr (GRAD_A)
      split_slab<SelfSplitT, SelfSplitT>(self_split_rows(smem, buf), self_split_cols(smem, buf), wr0, wc0, wave, lane, acc);
    else
      split_slab<SelfSplitS, SelfSplitS>(self_split_rows(smem, buf), self_split_cols(smem, buf), wr0, wc0, wave, lane, acc);
  };
  // Slab s is formed and staged while slab s-1 is multiplied, so the products start as soon as
  // the first pieces have arrived; the guard's answer is only needed before the results are
  // stored (an item that fails it has been multiplied in vain).
  static_for<0, kSelfSlabs>([&](auto sc_) __attribute__((always_inline)) {
    constexpr int s = decltype(sc_)::value;
    if constexpr (s < kSelfSlabs) {
      if (!RAGGED || s < slabs) {
        make_h(sc_);
        if constexpr (s + kAhead < kSelfSlabs) load_y(std::integral_constant<int, s + kAhead>{});
        make_y(sc_);
#pragma unroll
        for (int l = 0; l < 2; ++l) {
          if constexpr (SPLIT) {
            if constexpr (GRAD_A) {
              SelfSplitT::put(self_split_rows(smem, s & 1), tid, l, rg[s][l]);
              SelfSplitT::put(self_split_cols(smem, s & 1), tid, l, ry[s][l]);
            }
          } else if constexpr (GRAD_A) {  // rows <- H[m][n], columns <- EB[k][n]
            ST::put(Rs[s & 1], tid, l, rg[s][l]);
            ST::put(Cs[s & 1], tid, l, ry[s][l]);
          } else {                 // rows <- EA[m][k], columns <- H[m][n]
            SP::put(Rs[s & 1], tid, l, ry[s][l]);
            SP::put(Cs[s & 1], tid, l, rg[s][l]);
          }
        }
        if constexpr (SPLIT && !GRAD_A) {
          SelfSplitS::put(self_split_rows(smem, s & 1), tid, ry[s][0], ry[s][1]);
          SelfSplitS::put(self_split_cols(smem, s & 1), tid, rg[s][0], rg[s][1]);
        }
      }
    }
    if constexpr (s > 0) {
      if (!RAGGED || s <= slabs) multiply((s - 1) & 1);
    }
    __syncthreads();
  });
  if (!RAGGED || slabs == kSelfSlabs) multiply((kSelfSlabs - 1) & 1);
  bad = __builtin_amdgcn_readfirstlane(__syncthreads_or(bad));
  if (bad) {
    self_bwd_exact<GRAD_A>(p, batch, smem);
    return;
  }

  // grad = exp(x - shift) * acc, x = a (shift alpha per row) or b (beta per column)
  const int lr = lane >> 4, lc = (lane & 15) * 4;
  const long ubase = ((long)batch * R + wr0 + lr) * Cc + wc0 + lc;
  const elem_t* xb = (GRAD_A ? p.a : p.b) + ubase;
  elem_t* gp = p.grad + ubase;
  const int cc = RAGGED ? clamp4(Cc - (wc0 + lc)) : 4;
  const bool cok = cc > 0;
  const int rows_left = R - wr0 - lr;
  const float4 be4 = *reinterpret_cast<const float4*>(&s_be[wc0 + lc]);
  const float* alw = s_al + wr0 + lr;
  float4 xq[2][4];
  auto fetch = [&](int q) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (!RAGGED) xq[q & 1][t] = ld4(xb + (long)(16 * q + 4 * t) * Cc);
      else if (cok && 16 * q + 4 * t < rows_left) xq[q & 1][t] = ld4m(xb + (long)(16 * q + 4 * t) * Cc, cc, 0.f);
    }
  };
  fetch(0);
  acc_rows(acc, smem + wave * kStripFloats, lane,
           [&](int q) __attribute__((always_inline)) { if (q + 1 < 4) fetch(q + 1); },
           [&](int q, int t, float4 v) __attribute__((always_inline)) {
             const int ru = 16 * q + 4 * t;
             if (RAGGED && !(cok && ru < rows_left)) return;
             const float4 x = xq[q & 1][t];
             float4 e;
             if constexpr (GRAD_A) e = exp4(x, alw[ru]);
             else e = exp4(x, be4);
             const float4 r = make_float4(e.x * v.x, e.y * v.y, e.z * v.z, e.w * v.w);
             if (RAGGED) st4m(gp + (long)ru * Cc, cc, r);
             else st4(gp + (long)ru * Cc, r);
           });
}

// Workgroups come in groups of 16: the first eight take grad_a of eight consecutive
// items, the next eight grad_b of the same items (workgroup w runs on XCD w mod 8).
// A gradient whose pointer is null is skipped.
template <bool RAGGED, bool SPLIT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void k_log_self_bwd(const LogBwdArgs pa, const LogBwdArgs pb, const float* __restrict__ stats,
                    const int* __restrict__ hdr, int B) {
  __shared__ __attribute__((aligned(16))) float smem[kSelfLds];
  __shared__ __attribute__((aligned(16))) float s_al[kSelfMax], s_be[kSelfMax];
  const int w = blockIdx.x;
  const int item = (w >> 4) * 8 + (w & 7);
  if (item >= B) return;
  if (((w >> 3) & 1) == 0) {
    if (pa.grad) log_self_bwd_tile<true, RAGGED, SPLIT>(smem, s_al, s_be, pa, stats, hdr, item);
  } else {
    if (pb.grad) log_self_bwd_tile<false, RAGGED, SPLIT>(smem, s_al, s_be, pb, stats, hdr, item);
  }
}

}  // namespace GENBMM_NS
