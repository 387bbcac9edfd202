// Factored logbmm on the bf16 matrix instruction with fp32 accuracy: every staged factor
// x (fp32) is cut into three bfloat16 parts h + m + l = x exactly (h = x rounded to bf16,
// m = x - h rounded, l = the rest: 8 + 8 + 8 significant bits), and a product x y is taken
// as the six partial products h h, h m, m h, m m, h l, l h on v_mfma_f32_32x32x16_bf16
// (fp32 accumulate; bf16 x bf16 is exact in fp32).  What is left out - m l, l m, l l - is
// below 2^-23 of x y, the size of one fp32 rounding of the product itself.  The
// instruction does 16 reduction steps in the time the fp32 one (v_mfma_f32_32x32x2_f32)
// needs for one, so six of them per 16 steps are 2.7 times less matrix-pipe time, and -
// unlike the fp32 matrix instruction on this part - vector instructions of other waves can
// execute beside them (the counters show it for about a third of the pipe's busy cycles).
//
// Same tiles, guards, flags, epilogues and fix-up launches as the fp32 kernels of
// logbmm_mfma.h (a 64 x 64 block per wave as 2 x 2 accumulators, whose layout is that of
// the fp32 instruction; reduction in slabs of 16 through two LDS buffers); what differs is
// the staged form and the inner loop.  Ragged edges are a second instantiation of each
// kernel (RAGGED), handled as in logbmm_mfma.h: lines of a tile beyond the matrix re-read
// the last line (under a shift that makes the factor vanish where the line feeds stored
// results), stores are masked.  The forward takes any sizes: pieces that straddle the right
// edge are read element by element, the reduction tail is filled by the loader of the last
// slab.  The backward takes any M but K and N in multiples of four (no piece straddles an
// edge), and its partial last slab is a step of its own behind the loop.
//
// LDS layouts, three planes (h, m, l) per operand, words of two bf16:
//  * an operand whose source is [line][reduction] (reduction contiguous): plane[line][8
//    words]; a lane stages four consecutive reduction steps of a line (one 8-byte store
//    per plane) and reads the eight steps of its line that the instruction wants from it
//    as one 16-byte load.
//  * an operand whose source is [reduction][line]: plane[8 step pairs][lines + 8]; a lane
//    stages a pair of reduction steps for LW consecutive lines (the pair shares a word;
//    one store of LW words per plane) and reads its eight steps as four words a row apart.
#pragma once

#include "logbmm_mfma.h"
#include "split_bf16.h"

namespace GENBMM_NS {

// source [line][reduction]
template <int OUT, int NT>
struct SplitT {
  static constexpr int PLANE = OUT * 8;      // words
  static constexpr int BUF = 3 * PLANE;
  static constexpr int PER = OUT * 4 / NT;   // pieces (a line, four reduction steps) per thread
  static_assert(PER >= 1 && OUT * 4 % NT == 0, "");
  static __device__ __forceinline__ int line(int tid, int l) { return (tid >> 2) + l * (NT / 4); }
  static __device__ __forceinline__ int quad(int tid) { return tid & 3; }
  static __device__ __forceinline__ void put(unsigned* __restrict__ buf, int tid, int l, float4 v) {
    unsigned h0, m0, l0, h1, m1, l1;
    split2(v.x, v.y, h0, m0, l0);
    split2(v.z, v.w, h1, m1, l1);
    unsigned* p = buf + line(tid, l) * 8 + quad(tid) * 2;
    uintx2 w;
    w.x = h0; w.y = h1; *reinterpret_cast<uintx2*>(p) = w;
    w.x = m0; w.y = m1; *reinterpret_cast<uintx2*>(p + PLANE) = w;
    w.x = l0; w.y = l1; *reinterpret_cast<uintx2*>(p + 2 * PLANE) = w;
  }
  // the lane's operand of one 32-line block: line0 + lane % 32, reduction steps 8 (lane / 32) .. + 7
  static __device__ __forceinline__ bf16x8 frag(const unsigned* __restrict__ buf, int plane, int line0, int lane) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uintx4*>(buf + plane * PLANE + (line0 + (lane & 31)) * 8 +
                                                                       (lane >> 5) * 4));
  }
};

// source [reduction][line]
template <int OUT, int NT>
struct SplitS {
  static constexpr int LD = OUT + 8;         // words per step pair (lanes 32.. read four rows on: other banks)
  static constexpr int PLANE = 8 * LD;
  static constexpr int BUF = 3 * PLANE;
  static constexpr int LW = OUT * 8 / NT;    // lines per piece (a pair of reduction steps, LW lines); one piece per thread
  static_assert(LW == 2 || LW == 4, "");
  static constexpr int Q = OUT / LW;         // pieces per step pair
  static __device__ __forceinline__ int pair(int tid) { return tid / Q; }          // reduction steps 2 pair, 2 pair + 1
  static __device__ __forceinline__ int line0(int tid) { return (tid % Q) * LW; }
  static __device__ __forceinline__ void put(unsigned* __restrict__ buf, int tid, const float (&even)[LW],
                                             const float (&odd)[LW]) {
    unsigned h[LW], m[LW], l[LW];
#pragma unroll
    for (int j = 0; j < LW; ++j) split2(even[j], odd[j], h[j], m[j], l[j]);
    unsigned* p = buf + pair(tid) * LD + line0(tid);
    if constexpr (LW == 4) {
      uintx4 w;
      w.x = h[0]; w.y = h[1]; w.z = h[2]; w.w = h[3]; *reinterpret_cast<uintx4*>(p) = w;
      w.x = m[0]; w.y = m[1]; w.z = m[2]; w.w = m[3]; *reinterpret_cast<uintx4*>(p + PLANE) = w;
      w.x = l[0]; w.y = l[1]; w.z = l[2]; w.w = l[3]; *reinterpret_cast<uintx4*>(p + 2 * PLANE) = w;
    } else {
      uintx2 w;
      w.x = h[0]; w.y = h[1]; *reinterpret_cast<uintx2*>(p) = w;
      w.x = m[0]; w.y = m[1]; *reinterpret_cast<uintx2*>(p + PLANE) = w;
      w.x = l[0]; w.y = l[1]; *reinterpret_cast<uintx2*>(p + 2 * PLANE) = w;
    }
  }
  static __device__ __forceinline__ void put(unsigned* __restrict__ buf, int tid, float4 even, float4 odd) {
    static_assert(LW == 4, "");
    const float e[4] = {even.x, even.y, even.z, even.w}, o[4] = {odd.x, odd.y, odd.z, odd.w};
    put(buf, tid, e, o);
  }
  static __device__ __forceinline__ bf16x8 frag(const unsigned* __restrict__ buf, int plane, int line0, int lane) {
    const unsigned* p = buf + plane * PLANE + (lane >> 5) * 4 * LD + line0 + (lane & 31);
    uintx4 w;
    w.x = p[0]; w.y = p[LD]; w.z = p[2 * LD]; w.w = p[3 * LD];
    return __builtin_bit_cast(bf16x8, w);
  }
};

// LW consecutive elements as floats
template <int LW>
__device__ __forceinline__ void ldw(const elem_t* p, float (&v)[LW]) {
  if constexpr (LW == 4) {
    const float4 t = ld4(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else {
    typedef elem_t e2u __attribute__((ext_vector_type(2), aligned(sizeof(elem_t))));
    const e2u t = *reinterpret_cast<const e2u*>(p);
    v[0] = (float)t.x; v[1] = (float)t.y;
  }
}

// the first cnt of them (<= 0: none), `fill` for the rest
template <int LW>
__device__ __forceinline__ void ldwm(const elem_t* p, int cnt, float fill, float (&v)[LW]) {
  if (cnt >= LW) {
    ldw<LW>(p, v);
    return;
  }
#pragma unroll
  for (int j = 0; j < LW; ++j) v[j] = j < cnt ? (float)p[j] : fill;
}
__device__ __forceinline__ int clampw(int x, int w) { return min(max(x, 0), w); }

// The waves of a SIMD (waves i, i + 4, ... of the workgroup) run their matrix instructions at
// different priorities, all above the priority of staging: behind a barrier they would otherwise
// take turns instruction by instruction, finish their products together and then all stage at
// once with the matrix pipe idle; this way the first is through early and stages - vector work,
// which issues beside the others' matrix instructions - while the next one multiplies.
__device__ __forceinline__ void mfma_prio(int wave) {
  switch ((wave >> 2) & 3) {
    case 0: __builtin_amdgcn_s_setprio(3); break;
    case 1: __builtin_amdgcn_s_setprio(2); break;
    case 2: __builtin_amdgcn_s_setprio(1); break;
    default: __builtin_amdgcn_s_setprio(1); break;
  }
}

// The six partial products of one staged slab, for the wave's 2 x 2 blocks.  Products of one
// kind go to the four accumulators in turn (no instruction waits for the one before it);
// the small ones first.
template <class SR, class SC>
__device__ __forceinline__ void split_slab(const unsigned* __restrict__ R, const unsigned* __restrict__ Cs, int wr0,
                                           int wc0, int wave, int lane, floatx16 (&acc)[2][2]) {
  // Operand registers are asked for a phase ahead of their products and given up after them
  // (at most 40 of them live beside the 64 accumulators; the fences keep the compiler from
  // asking for all twelve operands up front).
  bf16x8 rh[2], ch[2], cl[2], rl[2], rm[2], cm[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    rh[i] = SR::frag(R, 0, wr0 + 32 * i, lane);
    cl[i] = SC::frag(Cs, 2, wc0 + 32 * i, lane);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    ch[i] = SC::frag(Cs, 0, wc0 + 32 * i, lane);
    rl[i] = SR::frag(R, 2, wr0 + 32 * i, lane);
  }
  __builtin_amdgcn_sched_barrier(0);
  mfma_prio(wave);
#pragma unroll
  for (int x = 0; x < 4; ++x) acc[x >> 1][x & 1] = mfma_bf16(rh[x >> 1], cl[x & 1], acc[x >> 1][x & 1]);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < 2; ++i) cm[i] = SC::frag(Cs, 1, wc0 + 32 * i, lane);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int x = 0; x < 4; ++x) acc[x >> 1][x & 1] = mfma_bf16(rl[x >> 1], ch[x & 1], acc[x >> 1][x & 1]);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < 2; ++i) rm[i] = SR::frag(R, 1, wr0 + 32 * i, lane);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int x = 0; x < 4; ++x) acc[x >> 1][x & 1] = mfma_bf16(rh[x >> 1], cm[x & 1], acc[x >> 1][x & 1]);
#pragma unroll
  for (int x = 0; x < 4; ++x) acc[x >> 1][x & 1] = mfma_bf16(rm[x >> 1], cm[x & 1], acc[x >> 1][x & 1]);
#pragma unroll
  for (int x = 0; x < 4; ++x) acc[x >> 1][x & 1] = mfma_bf16(rm[x >> 1], ch[x & 1], acc[x >> 1][x & 1]);
#pragma unroll
  for (int x = 0; x < 4; ++x) acc[x >> 1][x & 1] = mfma_bf16(rh[x >> 1], ch[x & 1], acc[x >> 1][x & 1]);
  __builtin_amdgcn_s_setprio(0);
  __builtin_amdgcn_sched_barrier(0);
}

// LDS words of a kernel on tile T whose row operand is staged by SR and column operand by SC
template <class SR, class SC>
constexpr int split_lds_words() { return 2 * (SR::BUF + SC::BUF); }

// The slab loop.  On entry slab 0 is loaded and staged (no barrier yet).
// The four waves of a SIMD (waves i, i + 4, i + 8, i + 12 of a workgroup of sixteen) issue their
// matrix instructions at descending priority (mfma_prio), so behind the barrier the first is
// through its products early and the last late.  The first half ("late" waves) stages the next
// slab behind its products, while the others still multiply; the second half ("early" waves),
// which must wait for the matrix pipe anyway, stages the next slab AHEAD of its products - from
// registers loaded a whole slab before - while the first half multiplies.  Nobody's staging is
// left for the end of the slab with the matrix pipe idle.  One load in flight per wave either way.
template <class Load, class Stage, class Mma>
__device__ __forceinline__ void split_loop(int slabs, bool early, Load&& load, Stage&& stage, Mma&& mma) {
  if (early && slabs > 1) load();
  __syncthreads();
  for (int s = 0; s < slabs; ++s) {
    const bool more = s + 1 < slabs;
    if (early) {
      if (more) stage((s + 1) & 1);
      if (s + 2 < slabs) load();
    } else {
      if (more) load();
    }
    mma(s & 1);
    if (!early && more) stage((s + 1) & 1);
    __syncthreads();
  }
}
// the second half of a workgroup's waves
template <int NT>
__device__ __forceinline__ bool split_early(int wave) { return wave >= NT / 128; }
// ----------------------------------------------------------------- forward
// rows <- EA from a[m][k] ([line][reduction]), columns <- EB from b[k][n] ([reduction][line]).
// Leaves the maxima, the tile flags and the header; KEEP: also the factors EA, EB (fp32, written
// by the tiles that stage them anyway: slab s of a row block's EA by its column block s mod
// tiles_n, likewise EB) and 1 / S, as k_log_fwd_mfma<T, RAGGED, true> does - what the sampling
// sweep reads.
// PIECES: the reduction axis is cut into `pieces` runs of slabs, each a workgroup of its own
// (workgroup = tile * pieces + piece); a piece leaves its sums S for its tile in ws_r
// ([piece][batch][M][N]) and k_log_fwd_join adds them, tests the guard and takes the logarithm.
// For problems with few output tiles and a long reduction, which would otherwise run on a few
// compute units.
template <class T, bool RAGGED, bool KEEP, bool PIECES = false>
__global__ __launch_bounds__(T::NT) __attribute__((amdgpu_waves_per_eu(T::WPE, T::WPE)))
void k_log_fwd_split(const elem_t* __restrict__ a, const elem_t* __restrict__ b, elem_t* __restrict__ out,
                     const float* __restrict__ stats, int* __restrict__ flags, float* __restrict__ ws_ea,
                     float* __restrict__ ws_eb, float* __restrict__ ws_r, int* __restrict__ ws_hdr, int M, int K,
                     int N, int tiles_m, int tiles_n, int pieces = 1) {
  static_assert(!PIECES || (RAGGED && !KEEP), "");
  constexpr int NT = T::NT;
  using SA = SplitT<T::TR, NT>;
  using SB = SplitS<T::TC, NT>;
  constexpr int LW = SB::LW;
  extern __shared__ __attribute__((aligned(16))) unsigned split_smem[];
  static_assert(split_lds_words<SA, SB>() >= (NT / 64) * kStripFloats, "");
  auto As = [&](int buf) __attribute__((always_inline)) { return split_smem + buf * SA::BUF; };
  auto Bs = [&](int buf) __attribute__((always_inline)) { return split_smem + 2 * SA::BUF + buf * SB::BUF; };
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / T::WC) * 64, wn0 = (wave % T::WC) * 64;
  const int per = tiles_m * tiles_n, wg = xcd_tile_id();
  const int tile = PIECES ? wg / pieces : wg, piece = PIECES ? wg - tile * pieces : 0;
  const int batch = tile / per, rem = tile - batch * per;
  const int m0 = (rem / tiles_n) * T::TR, n0 = (rem % tiles_n) * T::TC;
  const float* st = stats + (long)batch * (M + N);
  // the slabs of this workgroup: all of them, or the piece's run (no piece is empty)
  const int slabs_all = RAGGED ? (K + kMS - 1) / kMS : K / kMS;
  const int slabs_piece = PIECES ? (slabs_all + pieces - 1) / pieces : slabs_all;
  const int slab0 = piece * slabs_piece;

  // a pieces: line m0 + line(l), four k from quad * 4;  the b piece: rows 2 pair, 2 pair + 1 of the
  // slab, LW columns from bcol
  const elem_t* pa[SA::PER];
  float al[SA::PER];
  bool va[SA::PER];
#pragma unroll
  for (int l = 0; l < SA::PER; ++l) {
    const int line = m0 + SA::line(tid, l);
    va[l] = !RAGGED || line < M;
    pa[l] = a + ((long)batch * M + (va[l] ? line : M - 1)) * K + SA::quad(tid) * 4 + (long)slab0 * kMS;
    al[l] = va[l] ? st[line] : INFINITY;  // lines beyond the matrix: exp -> 0
  }
  // the factors live at the same offsets in their own arrays (the source pointers run one slab
  // ahead of what is being staged, whichever side of its products a wave stages on)
  const int nblk = rem % tiles_n, mblk = rem / tiles_n;
  const long da = KEEP ? ws_distance(ws_ea, a) - 4l * kMS : 0, db = KEEP ? ws_distance(ws_eb, b) - 4l * kMS * N : 0;
  int s_stage = 0, sa = 0, sb = 0;  // the slab the next stage() forms; s_stage mod tiles_n, mod tiles_m
  const int bcol = n0 + SB::line0(tid);
  const int cb = RAGGED ? clampw(N - bcol, LW) : LW;  // columns of the b piece inside the matrix
  const int brow = 2 * SB::pair(tid);
  const elem_t* pb = b + ((long)batch * K + brow + (long)slab0 * kMS) * N + (cb > 0 ? bcol : 0);
  float be[LW];
#pragma unroll
  for (int j = 0; j < LW; ++j) be[j] = j < cb ? st[M + bcol + j] : INFINITY;
  if (!PIECES && tile == 0 && tid == 0) {
    ws_hdr[1] = T::TR;
    ws_hdr[2] = T::TC;
    ws_hdr[0] = KEEP ? kWsMfma : kWsFast;
  }

  floatx16 acc[2][2];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[x >> 1][x & 1][i] = 0.f;

  const int slabs = PIECES ? min(slabs_piece, slabs_all - slab0) : slabs_all;
  // reduction steps of a partial last slab (of the last piece)
  const int ktail = RAGGED && (!PIECES || slab0 + slabs == slabs_all) ? K % kMS : 0;
  int s_load = 0;                                  // the slab the next load() fetches
  float4 ra[SA::PER];
  float rbe[LW], rbo[LW];
  auto load = [&]() __attribute__((always_inline)) {
    if (RAGGED && ktail != 0 && s_load == slabs - 1) {
      const int ca = clamp4(ktail - SA::quad(tid) * 4);
#pragma unroll
      for (int l = 0; l < SA::PER; ++l) ra[l] = ld4m(pa[l], ca, -INFINITY);
      ldwm<LW>(pb, brow < ktail ? cb : 0, -INFINITY, rbe);
      ldwm<LW>(pb + N, brow + 1 < ktail ? cb : 0, -INFINITY, rbo);
    } else {
#pragma unroll
      for (int l = 0; l < SA::PER; ++l) ra[l] = ld4(pa[l]);
      if (RAGGED) {
        ldwm<LW>(pb, cb, -INFINITY, rbe);
        ldwm<LW>(pb + N, cb, -INFINITY, rbo);
      } else {
        ldw<LW>(pb, rbe);
        ldw<LW>(pb + N, rbo);
      }
    }
#pragma unroll
    for (int l = 0; l < SA::PER; ++l) pa[l] += kMS;
    pb += (long)kMS * N;
    ++s_load;
  };
  auto stage = [&](int buf) __attribute__((always_inline)) {
    const bool tail = RAGGED && ktail != 0 && s_stage == slabs - 1;
#pragma unroll
    for (int l = 0; l < SA::PER; ++l) {
      const float4 e = exp4(ra[l], al[l]);
      SA::put(As(buf), tid, l, e);
      if (KEEP && sa == nblk) {
        if (!RAGGED) st4(ws_twin(pa[l], da), e);
        else if (va[l]) st4m(ws_twin(pa[l], da), tail ? clamp4(ktail - SA::quad(tid) * 4) : 4, e);
      }
    }
    float ee[LW], eo[LW];
#pragma unroll
    for (int j = 0; j < LW; ++j) {
      ee[j] = exp_st(rbe[j] - be[j]);
      eo[j] = exp_st(rbo[j] - be[j]);
    }
    SB::put(Bs(buf), tid, ee, eo);
    if (KEEP && sb == mblk) {
      float* we = ws_twin(pb, db);
#pragma unroll
      for (int j = 0; j < LW; ++j) {
        if (j < cb && (!tail || brow < ktail)) we[j] = ee[j];
        if (j < cb && (!tail || brow + 1 < ktail)) we[N + j] = eo[j];
      }
    }
    if (KEEP) {
      ++s_stage;
      sa = sa + 1 == tiles_n ? 0 : sa + 1;
      sb = sb + 1 == tiles_m ? 0 : sb + 1;
    }
  };

  load();
  stage(0);
  split_loop(slabs, split_early<NT>(wave), load, stage, [&](int buf) __attribute__((always_inline)) {
    split_slab<SA, SB>(As(buf), Bs(buf), wm0, wn0, wave, lane, acc);
  });

  if constexpr (PIECES) {  // the piece's sums, row-wise; the guard is k_log_fwd_join's
    __syncthreads();       // every wave is done with the staging buffers
    const int lr = lane >> 4, lc = (lane & 15) * 4;
    const int cc = clamp4(N - (n0 + wn0 + lc));
    const long ubase = (((long)piece * (gridDim.x / (pieces * per)) + batch) * M + m0 + wm0) * N + n0 + wn0;
    const int voff = lr * N + lc, rows_left = M - (m0 + wm0) - lr;
    acc_rows(acc, reinterpret_cast<float*>(split_smem) + wave * kStripFloats, lane, [](int) {},
             [&](int q, int t, float4 sv) __attribute__((always_inline)) {
               const int ru = 16 * q + 4 * t;
               if (cc > 0 && ru < rows_left) st4m(ws_r + ubase + (long)ru * N + voff, cc, sv);
             });
    return;
  }
  // guard (as k_log_fwd_mfma): S >= 2^-40 and finite; every shift finite and not below the floor;
  // no shift below -30 opposite a row or column at the floor
  const float thr = fast_exp2(-kMfmaGuardBits);
  int bad = 0;
  {
    const int rlim = M - (m0 + wm0) - mfma_row_l(lane);   // rows of this lane below rlim exist
    const int clim = N - (n0 + wn0) - (lane & 31);        // column blocks at offset < clim exist
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float s = acc[x >> 1][x & 1][i];
        const bool here = !RAGGED || ((x >> 1) * 32 + mfma_row_u(i) < rlim && (x & 1) * 32 < clim);
        if (here && !((s >= thr) && (s < INFINITY))) bad = 1;
      }
  }
  static_assert(T::TR + T::TC <= NT, "one shift per thread");
  int low = 0, neg = 0;  // bit 0: of a row, bit 1: of a column
  {
    const bool row = tid < T::TR;
    const bool here = tid < T::TR + T::TC && (!RAGGED || (row ? m0 + tid < M : n0 + tid - T::TR < N));
    if (here) {
      const float sh = row ? st[m0 + tid] : st[M + n0 + tid - T::TR];
      if (!((sh >= kFloor) && (sh < INFINITY))) bad = 1;
      if (sh <= 0.45f * kFloor) low = row ? 1 : 2;
      if (sh < -30.f) neg = row ? 1 : 2;
    }
  }
  const int row_low = __syncthreads_or(low & 1), col_low = __syncthreads_or(low & 2);
  if (row_low | col_low) {  // uniform, and rare
    const int row_neg = __syncthreads_or(neg & 1), col_neg = __syncthreads_or(neg & 2);
    if ((row_low && col_neg) || (col_low && row_neg)) bad = 1;
  }
  bad = __syncthreads_or(bad);  // also: every wave is done with the staging buffers
  if (tid == 0) flags[tile] = bad;
  if (bad) return;  // the fix-up launch recomputes this tile

  // out = log S + alpha + beta, written row-wise
  const int lr = lane >> 4, lc = (lane & 15) * 4;
  const int cc = RAGGED ? clamp4(N - (n0 + wn0 + lc)) : 4;  // columns of this lane's pieces that exist
  const bool cok = cc > 0;
  const float4 be4 = RAGGED ? ld4m(st + M + (cok ? n0 + wn0 + lc : 0), cc, 0.f) : ld4(st + M + n0 + wn0 + lc);
  const float* alw = st + m0 + wm0 + lr;
  const long ubase = ((long)batch * M + m0 + wm0) * N + n0 + wn0;
  const int voff = lr * N + lc;
  const int rows_left = M - (m0 + wm0) - lr;
  acc_rows(acc, reinterpret_cast<float*>(split_smem) + wave * kStripFloats, lane, [](int) {},
           [&](int q, int t, float4 sv) __attribute__((always_inline)) {
             const int ru = 16 * q + 4 * t;
             if (RAGGED && !(cok && ru < rows_left)) return;
             const float alr = alw[ru];
             const float4 ov = make_float4(__builtin_fmaf(fast_log2(sv.x), kLn2, alr + be4.x),
                                           __builtin_fmaf(fast_log2(sv.y), kLn2, alr + be4.y),
                                           __builtin_fmaf(fast_log2(sv.z), kLn2, alr + be4.z),
                                           __builtin_fmaf(fast_log2(sv.w), kLn2, alr + be4.w));
             if (RAGGED) st4m(out + ubase + (long)ru * N + voff, cc, ov);
             else st4(out + ubase + (long)ru * N + voff, ov);
             if constexpr (KEEP) {
               const float4 rv = make_float4(__builtin_amdgcn_rcpf(sv.x), __builtin_amdgcn_rcpf(sv.y),
                                             __builtin_amdgcn_rcpf(sv.z), __builtin_amdgcn_rcpf(sv.w));
               if (RAGGED) st4m(ws_r + ubase + (long)ru * N + voff, cc, rv);
               else st4(ws_r + ubase + (long)ru * N + voff, rv);
             }
           });
}

// The pieces of k_log_fwd_split<.., PIECES> joined: S = the sum of the pieces' sums for a cell, then
// the forward's guard - per tile of TR x TC cells, the tile shape that the flags, the header and the
// exact fix-up launch behind this kernel go by - and out = log S + alpha + beta.  One workgroup per tile.
template <int TR, int TC>
__global__ __launch_bounds__(256) void k_log_fwd_join(const float* __restrict__ parts, elem_t* __restrict__ out,
                                                      const float* __restrict__ stats, int* __restrict__ flags,
                                                      int* __restrict__ ws_hdr, int B, int M, int N, int tiles_m,
                                                      int tiles_n, int pieces) {
  const int tid = threadIdx.x, tile = blockIdx.x, per = tiles_m * tiles_n;
  const int batch = tile / per, rem = tile - batch * per;
  const int m0 = (rem / tiles_n) * TR, n0 = (rem % tiles_n) * TC;
  const float* st = stats + (long)batch * (M + N);
  const long piece_stride = (long)B * M * N;
  const float thr = fast_exp2(-kMfmaGuardBits);
  int bad = 0, low = 0, neg = 0;  // bit 0: of a row, bit 1: of a column
  for (int c = tid; c < TR * (TC / 4); c += 256) {
    const int m = m0 + c / (TC / 4), n = n0 + (c % (TC / 4)) * 4;
    const int cc = clamp4(N - n);
    if (m >= M || cc <= 0) continue;
    const long at = ((long)batch * M + m) * N + n;
    float4 sv = ld4m(parts + at, cc, 0.f);
    int p = 1;
    for (; p + 8 <= pieces; p += 8) {  // eight pieces' loads in flight; added in the pieces' order
      float4 x[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) x[q] = ld4m(parts + (p + q) * piece_stride + at, cc, 0.f);
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        sv.x += x[q].x; sv.y += x[q].y; sv.z += x[q].z; sv.w += x[q].w;
      }
    }
    for (; p < pieces; ++p) {
      const float4 x = ld4m(parts + p * piece_stride + at, cc, 0.f);
      sv.x += x.x; sv.y += x.y; sv.z += x.z; sv.w += x.w;
    }
    const float alr = st[m];
    const float4 be4 = ld4m(st + M + n, cc, 0.f);
    const float s4[4] = {sv.x, sv.y, sv.z, sv.w}, b4[4] = {be4.x, be4.y, be4.z, be4.w};
    if (!((alr >= kFloor) && (alr < INFINITY))) bad = 1;
    if (alr <= 0.45f * kFloor) low |= 1;
    if (alr < -30.f) neg |= 1;
    float o4[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      o4[j] = 0.f;
      if (j < cc) {
        if (!((s4[j] >= thr) && (s4[j] < INFINITY)) || !((b4[j] >= kFloor) && (b4[j] < INFINITY))) bad = 1;
        if (b4[j] <= 0.45f * kFloor) low |= 2;
        if (b4[j] < -30.f) neg |= 2;
        o4[j] = __builtin_fmaf(fast_log2(s4[j]), kLn2, alr + b4[j]);
      }
    }
    st4m(out + at, cc, make_float4(o4[0], o4[1], o4[2], o4[3]));
  }
  const int row_low = __syncthreads_or(low & 1), col_low = __syncthreads_or(low & 2);
  const int row_neg = __syncthreads_or(neg & 1), col_neg = __syncthreads_or(neg & 2);
  if ((row_low && col_neg) || (col_low && row_neg)) bad = 1;
  bad = __syncthreads_or(bad);
  if (tid == 0) flags[tile] = bad;  // the fix-up launch recomputes a flagged tile
  if (tile == 0 && tid == 0) {
    ws_hdr[1] = TR;
    ws_hdr[2] = TC;
    ws_hdr[0] = kWsFast;
  }
}

// ------------------------------------------------------- sampling sweep
// The sampling sweep described in logbmm_mfma.h: the forward's contraction again on its fp32
// factors EA, EB - cut into their three parts while they are staged, no exponential - with the
// accumulators started at -t, t = u S the cell's target; after every slab of 16 terms a
// register per cell keeps, by a signed-integer minimum over (value with its low six bits
// replaced by 62 - slab; seven bits and 126 - slab for more than 62 slabs: `tmask` = 63 or 127),
// the slab in which the prefix sum passes t and -rem at the start of that slab.  S is the reciprocal of the forward's 1 / S, the targets are shrunk by 2^-22;
// results: the code -2 - slab in idx, rem in `remw`.  The partial products are added in the
// forward's order, so the sums the sweep compares with its targets are the forward's.  A tile
// with a cell whose S is below 2^-40 or not finite, or that lies in a tile the forward
// flagged, sets that flag and leaves: the forward's tile is redone exactly.  128 x 128 tiles of
// four waves with 256 registers (64 accumulators and 64 history registers per lane); always
// the any-size form of the loaders.
template <class T>
__global__ __launch_bounds__(T::NT) __attribute__((amdgpu_waves_per_eu(2, 2)))
void k_sample_sweep_split(const float* __restrict__ ws_ea, const float* __restrict__ ws_eb,
                          const elem_t* __restrict__ out, const float* __restrict__ stats,
                          int* __restrict__ flags, float* __restrict__ remw, int32_t* __restrict__ idx,
                          uint64_t seed, uint64_t offset, int M, int K, int N, int tiles_m, int tiles_n, int ftr,
                          int ftc, int ftiles_m, int ftiles_n, int tmask) {
  constexpr bool RAGGED = true;
  constexpr int NT = T::NT;
  using SA = SplitT<T::TR, NT>;
  using SB = SplitS<T::TC, NT>;
  static_assert(SB::LW == 4, "");
  __shared__ __attribute__((aligned(16))) unsigned smem[split_lds_words<SA, SB>()];
  auto As = [&](int buf) __attribute__((always_inline)) { return smem + buf * SA::BUF; };
  auto Bs = [&](int buf) __attribute__((always_inline)) { return smem + 2 * SA::BUF + buf * SB::BUF; };
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / T::WC) * 64, wn0 = (wave % T::WC) * 64;
  const int per = tiles_m * tiles_n, tile = xcd_tile_id();
  const int batch = tile / per, rem = tile - batch * per;
  const int m0 = (rem / tiles_n) * T::TR, n0 = (rem % tiles_n) * T::TC;
  const float* st = stats + (long)batch * (M + N);

  // ---- targets: -t = -u S per cell into `remw`, row by row, four adjacent cells per lane and
  // step (they share one Philox block when rows are a multiple of four cells); then the
  // accumulators pick their cells up in the matrix-core layout.  The flags are the forward's,
  // one per tile of ITS shape (ftr x ftc).
  int* flag = flags + (batch * ftiles_m + m0 / ftr) * ftiles_n + n0 / ftc;
  const float lim = kMfmaGuardBits * kLn2 + 1e-3f;
  int bad = *flag;
  {
    constexpr int QR = T::TC / 4;  // quads per tile row
    const bool blocks = (N & 3) == 0;
#pragma unroll 4
    for (int q = tid; q < T::TR * QR; q += NT) {
      const int r = q / QR, m = m0 + r, n = n0 + (q - r * QR) * 4;
      if (RAGGED && (m >= M || n >= N)) continue;
      const long cell = ((long)batch * M + m) * N + n;
      const int cn = RAGGED ? clamp4(N - n) : 4;
      float u[4];
      philox_uniform4((uint64_t)cell, blocks, seed, offset, u);
      const float alr = st[m];
      const float4 be4 = ld4m(st + M + n, cn, 0.f), o4 = ld4m(out + cell, cn, 0.f);
      const float4 r4 = ld4m(remw + cell, cn, 1.f);  // the forward's 1 / S
      const float bev[4] = {be4.x, be4.y, be4.z, be4.w}, ov[4] = {o4.x, o4.y, o4.z, o4.w};
      const float rv[4] = {r4.x, r4.y, r4.z, r4.w};
      float tv[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float e = alr + bev[j] - ov[j];  // -log S
        if (j < cn && (!(e <= lim) || !(e > -INFINITY))) bad = 1;
        tv[j] = -(u[j] * kSampleShrink) * __builtin_amdgcn_rcpf(rv[j]);
      }
      st4m(remw + cell, cn, make_float4(tv[0], tv[1], tv[2], tv[3]));
    }
  }
  bad = __syncthreads_or(bad);  // also: the tile's -t are visible to the whole workgroup
  if (bad) {
    if (tid == 0) *flag = 1;
    return;
  }
  floatx16 acc[2][2];
  int low[2][2][16];
  const int col = lane & 31;
#pragma unroll
  for (int br = 0; br < 2; ++br)
#pragma unroll
    for (int bc = 0; bc < 2; ++bc) {
      const int n = n0 + wn0 + bc * 32 + col;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = m0 + wm0 + br * 32 + mfma_row(i, lane);
        const bool ok = !RAGGED || (m < M && n < N);
        const float nt = ok ? remw[((long)batch * M + m) * N + n] : 0.f;
        acc[br][bc][i] = nt;
        low[br][bc][i] = __float_as_int(nt) | tmask;  // all tag bits set: no slab has ended below t
      }
    }

  // ---- staging of EA ([line][reduction]) and EB (pairs of reduction steps), zeros beyond the matrix
  const int bcol = n0 + SB::line0(tid);
  const int cb = clamp4(N - bcol);
  const int brow = 2 * SB::pair(tid);
  bool va[SA::PER];
  const float* pa[SA::PER];
#pragma unroll
  for (int l = 0; l < SA::PER; ++l) {
    const int line = m0 + SA::line(tid, l);
    va[l] = line < M;
    pa[l] = ws_ea + ((long)batch * M + (va[l] ? line : M - 1)) * K + SA::quad(tid) * 4;
  }
  const float* pb = ws_eb + ((long)batch * K + brow) * N + (cb > 0 ? bcol : 0);
  const int ktail = K % kMS;
  const int slabs = (K + kMS - 1) / kMS;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  float4 ra[SA::PER], rbe, rbo;
  int s_load = 0, s_mma = 0;
  auto load = [&]() __attribute__((always_inline)) {
    if (ktail != 0 && s_load == slabs - 1) {
      const int ca = clamp4(ktail - SA::quad(tid) * 4);
#pragma unroll
      for (int l = 0; l < SA::PER; ++l) ra[l] = va[l] ? ld4m(pa[l], ca, 0.f) : zero;
      rbe = brow < ktail ? ld4m(pb, cb, 0.f) : zero;
      rbo = brow + 1 < ktail ? ld4m(pb + N, cb, 0.f) : zero;
    } else {
#pragma unroll
      for (int l = 0; l < SA::PER; ++l) ra[l] = va[l] ? ld4(pa[l]) : zero;
      rbe = ld4m(pb, cb, 0.f);
      rbo = ld4m(pb + N, cb, 0.f);
    }
#pragma unroll
    for (int l = 0; l < SA::PER; ++l) pa[l] += kMS;
    pb += (long)kMS * N;
    ++s_load;
  };
  auto stage = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int l = 0; l < SA::PER; ++l) SA::put(As(buf), tid, l, ra[l]);
    SB::put(Bs(buf), tid, rbe, rbo);
  };
  load();
  stage(0);
  split_loop(slabs, split_early<NT>(wave), load, stage, [&](int buf) __attribute__((always_inline)) {
    split_slab<SA, SB>(As(buf), Bs(buf), wm0, wn0, wave, lane, acc);
    const int tag = tmask - 1 - s_mma;
    ++s_mma;
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int v = (__float_as_int(acc[x >> 1][x & 1][i]) & ~tmask) | (tag & tmask);  // one v_bfi_b32
        low[x >> 1][x & 1][i] = min(low[x >> 1][x & 1][i], v);
      }
  });

  // ---- slab in which the prefix passes t, and rem at its start
#pragma unroll
  for (int br = 0; br < 2; ++br)
#pragma unroll
    for (int bc = 0; bc < 2; ++bc) {
      const int n = n0 + wn0 + bc * 32 + col;
      if (RAGGED && n >= N) continue;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = m0 + wm0 + br * 32 + mfma_row(i, lane);
        if (RAGGED && m >= M) continue;
        const long cell = ((long)batch * M + m) * N + n;
        const int below = tmask - (low[br][bc][i] & tmask);
        // a target that the sums never reach lies within their rounding of the total: the last term
        idx[cell] = below >= slabs ? K - 1 : -2 - below;
        remw[cell] = -__int_as_float(low[br][bc][i] & ~tmask);
      }
    }
}

// ---------------------------------------------------------------- backward
// Operands formed from a, b, out, g and the maxima while they are staged (as
// log_bwd_mfma_tile_lean): EA = exp(a - alpha), EB = exp(b - beta), H = g exp(alpha + beta - out).
// GRAD_A: tile (m,k) of grad_a = EA * sum_n H[m][n] EB[k][n]; rows <- H, columns <- EB, both
//         sources [line][reduction].
// GRAD_B: tile (k,n) of grad_b = EB * sum_m EA[m][k] H[m][n]; rows <- EA, columns <- H, both
//         sources [reduction][line].
template <class T, bool GRAD_A>
struct SplitBwd {
  static constexpr int NT = T::NT;
  using SR = std::conditional_t<GRAD_A, SplitT<T::TR, NT>, SplitS<T::TR, NT>>;
  using SC = std::conditional_t<GRAD_A, SplitT<T::TC, NT>, SplitS<T::TC, NT>>;
  static constexpr int WORDS = split_lds_words<SR, SC>();
};

template <class T, bool GRAD_A, bool RAGGED>
__device__ __forceinline__ void log_bwd_split_tile(unsigned* __restrict__ smem, int tile, const elem_t* __restrict__ g,
                                                   const LeanSrc src, const int* __restrict__ ws_hdr,
                                                   const int* __restrict__ fwd_flags, elem_t* __restrict__ grad, int M,
                                                   int K, int N, int tiles_r, int tiles_c) {
  using W = SplitBwd<T, GRAD_A>;
  using SR = typename W::SR;
  using SC = typename W::SC;
  constexpr int NT = T::NT;
  static_assert(W::WORDS >= (NT / 64) * kStripFloats, "");
  auto Rs = [&](int buf) __attribute__((always_inline)) { return smem + buf * SR::BUF; };
  auto Cs = [&](int buf) __attribute__((always_inline)) { return smem + 2 * SR::BUF + buf * SC::BUF; };
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr0 = (wave / T::WC) * 64, wc0 = (wave % T::WC) * 64;
  const int per = tiles_r * tiles_c;
  const int batch = tile / per, rem = tile - batch * per;
  const int r0 = (rem / tiles_c) * T::TR, c0 = (rem % tiles_c) * T::TC;
  const int Q = GRAD_A ? N : M;
  const int R = GRAD_A ? M : K, Cc = GRAD_A ? K : N;
  const float* al = src.stats + (long)batch * (M + N);
  const float* be = al + M;
  floatx16 acc[2][2];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[x >> 1][x & 1][i] = 0.f;
  const int slabs = Q / kMS;                // whole slabs: the loop
  const int qtail = RAGGED ? Q % kMS : 0;   // reduction steps of a partial last slab: one more step behind the
                                            // loop, with a loader of its own (inside the loop's loader it cost
                                            // 19 spilled registers and the kernel ran 1.7 times slower)

  // Addresses are a base per workgroup (scalar registers, stepped slab by slab) plus a fixed
  // 32-bit offset per thread: the vector registers go to operands and accumulators.
  // RAGGED: any M; K and N multiples of four, so that no piece straddles the right edge of its
  // matrix (other shapes run their backward on the fp32 instruction).  Fills of the partial last
  // slab make a factor vanish: -inf for a and b, +inf for out, 0 for g.
  if constexpr (GRAD_A) {
    // rows: H pieces (line m, four n); columns: EB pieces (line k, four n); beta of the slab's four
    // columns is the same for every piece of a thread (all share their quad).  Lines beyond the
    // matrix re-read the last line: they only feed results that are not stored.
    const elem_t* ob = src.out + (long)batch * M * N;
    const elem_t* gb = g + (long)batch * M * N;
    const elem_t* bb = src.b + (long)batch * K * N;
    const float* beb = be;
    int oo[SR::PER], yo[SC::PER];
    float alh[SR::PER];
#pragma unroll
    for (int l = 0; l < SR::PER; ++l) {
      const int m = RAGGED ? min(r0 + SR::line(tid, l), M - 1) : r0 + SR::line(tid, l);
      oo[l] = m * N + SR::quad(tid) * 4;
      alh[l] = al[m];
    }
#pragma unroll
    for (int l = 0; l < SC::PER; ++l) {
      const int k = RAGGED ? min(c0 + SC::line(tid, l), K - 1) : c0 + SC::line(tid, l);
      yo[l] = k * N + SC::quad(tid) * 4;
    }
    const int beo = SR::quad(tid) * 4;
    float4 ro[SR::PER], rg[SR::PER], ry[SC::PER], bslab;
    auto load = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int l = 0; l < SC::PER; ++l) ry[l] = ld4(bb + yo[l]);
#pragma unroll
      for (int l = 0; l < SR::PER; ++l) {
        ro[l] = ld4(ob + oo[l]);
        rg[l] = ld4(gb + oo[l]);
      }
      bslab = ld4(beb + beo);
      ob += kMS; gb += kMS; bb += kMS; beb += kMS;
    };
    auto stage = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
      for (int l = 0; l < SC::PER; ++l) SC::put(Cs(buf), tid, l, exp4(ry[l], bslab));
#pragma unroll
      for (int l = 0; l < SR::PER; ++l) {
        const float4 sh = make_float4(alh[l] + bslab.x, alh[l] + bslab.y, alh[l] + bslab.z, alh[l] + bslab.w);
        SR::put(Rs(buf), tid, l, mul_exp4(rg[l], sh, ro[l]));
      }
    };
    load();
    if (bwd_tile_flagged(ws_hdr, fwd_flags, false, true, r0, T::TR, batch, M, N, tid, NT)) return;
    stage(0);
    split_loop(slabs, split_early<NT>(wave), load, stage, [&](int buf) __attribute__((always_inline)) {
      split_slab<SR, SC>(Rs(buf), Cs(buf), wr0, wc0, wave, lane, acc);
    });
    if (RAGGED && qtail != 0) {  // uniform
      const int left = qtail - beo;  // all pieces of a thread share their quad
#pragma unroll
      for (int l = 0; l < SC::PER; ++l) ry[l] = ld4m(bb + yo[l], left, -INFINITY);
#pragma unroll
      for (int l = 0; l < SR::PER; ++l) {
        ro[l] = ld4m(ob + oo[l], left, INFINITY);
        rg[l] = ld4m(gb + oo[l], left, 0.f);
      }
      bslab = ld4m(beb + beo, left, 0.f);
      stage(0);
      __syncthreads();
      split_slab<SR, SC>(Rs(0), Cs(0), wr0, wc0, wave, lane, acc);
      __syncthreads();
    }
  } else {
    // rows: EA pieces (steps m, m + 1; LW lines k); columns: H pieces (steps m, m + 1; LW lines n);
    // both operands' pieces of a thread are on the same pair of steps.  RAGGED: lines beyond the
    // matrix re-read the last LW lines - they only feed results that are not stored.
    constexpr int LR = SR::LW, LC = SC::LW;
    static_assert(SR::Q == SC::Q, "");
    const int m2 = 2 * SR::pair(tid);
    const elem_t* ab = src.a + (long)batch * M * K;
    const elem_t* ob = src.out + (long)batch * M * N;
    const elem_t* gb = g + (long)batch * M * N;
    const float* alb = al;
    const int kc = RAGGED ? min(r0 + SR::line0(tid), K - LR) : r0 + SR::line0(tid);
    const int nc = RAGGED ? min(c0 + SC::line0(tid), N - LC) : c0 + SC::line0(tid);
    const int yo = m2 * K + kc, oo = m2 * N + nc;
    float bec[LC];
#pragma unroll
    for (int j = 0; j < LC; ++j) bec[j] = be[nc + j];
    float ye[LR], yd[LR], oe[LC], od[LC], ge[LC], gd[LC];
    float a0, a1;
    auto load = [&]() __attribute__((always_inline)) {
      ldw<LR>(ab + yo, ye);
      ldw<LR>(ab + yo + K, yd);
      ldw<LC>(ob + oo, oe);
      ldw<LC>(ob + oo + N, od);
      ldw<LC>(gb + oo, ge);
      ldw<LC>(gb + oo + N, gd);
      a0 = alb[m2];
      a1 = alb[m2 + 1];
      ab += (long)kMS * K;
      ob += (long)kMS * N;
      gb += (long)kMS * N;
      alb += kMS;
    };
    auto stage = [&](int buf) __attribute__((always_inline)) {
      float e0[LR], e1[LR], h0[LC], h1[LC];
#pragma unroll
      for (int j = 0; j < LR; ++j) {
        e0[j] = exp_st(ye[j] - a0);
        e1[j] = exp_st(yd[j] - a1);
      }
#pragma unroll
      for (int j = 0; j < LC; ++j) {
        h0[j] = ge[j] * exp_st(a0 + bec[j] - oe[j]);
        h1[j] = gd[j] * exp_st(a1 + bec[j] - od[j]);
      }
      SR::put(Rs(buf), tid, e0, e1);
      SC::put(Cs(buf), tid, h0, h1);
    };
    load();
    if (bwd_tile_flagged(ws_hdr, fwd_flags, false, false, c0, T::TC, batch, M, N, tid, NT)) return;
    stage(0);
    split_loop(slabs, split_early<NT>(wave), load, stage, [&](int buf) __attribute__((always_inline)) {
      split_slab<SR, SC>(Rs(buf), Cs(buf), wr0, wc0, wave, lane, acc);
    });
    if (RAGGED && qtail != 0) {  // uniform; steps beyond M re-read row M - 1 and are replaced by the fills
      const int c0r = min(m2, qtail - 1), c1r = min(m2 + 1, qtail - 1);
      ldw<LR>(ab + c0r * K + kc, ye);
      ldw<LR>(ab + c1r * K + kc, yd);
      ldw<LC>(ob + c0r * N + nc, oe);
      ldw<LC>(ob + c1r * N + nc, od);
      ldw<LC>(gb + c0r * N + nc, ge);
      ldw<LC>(gb + c1r * N + nc, gd);
      a0 = alb[c0r];
      a1 = alb[c1r];
      const bool in0 = m2 < qtail, in1 = m2 + 1 < qtail;
#pragma unroll
      for (int j = 0; j < LR; ++j) {
        ye[j] = in0 ? ye[j] : -INFINITY;
        yd[j] = in1 ? yd[j] : -INFINITY;
      }
#pragma unroll
      for (int j = 0; j < LC; ++j) {
        ge[j] = in0 ? ge[j] : 0.f;
        gd[j] = in1 ? gd[j] : 0.f;
      }
      stage(0);
      __syncthreads();
      split_slab<SR, SC>(Rs(0), Cs(0), wr0, wc0, wave, lane, acc);
      __syncthreads();
    }
  }

  // grad = EX * acc with EX = exp(a - alpha) (grad_a) or exp(b - beta) (grad_b), row-wise
  const int lr = lane >> 4, lc = (lane & 15) * 4;
  const int voff = lr * Cc + lc;
  const long ubase = ((long)batch * R + r0 + wr0) * Cc + c0 + wc0;
  const elem_t* xb = (GRAD_A ? src.a : src.b) + ubase + voff;
  elem_t* gp = grad + ubase + voff;
  const int cc = RAGGED ? clamp4(Cc - (c0 + wc0 + lc)) : 4;
  const bool cok = cc > 0;
  const int rows_left = R - (r0 + wr0) - lr;
  float4 becol = make_float4(0.f, 0.f, 0.f, 0.f);
  if constexpr (!GRAD_A) becol = RAGGED ? ld4m(be + (cok ? c0 + wc0 + lc : 0), cc, 0.f) : ld4(be + c0 + wc0 + lc);
  const float* alrow = al + r0 + wr0 + lr;
  float4 xq[2][4];
  float xa[2][4];
  auto fetch = [&](int q) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const bool live = !RAGGED || (cok && 16 * q + 4 * t < rows_left);
      if (live) {
        xq[q & 1][t] = RAGGED ? ld4m(xb + (long)(16 * q + 4 * t) * Cc, cc, -INFINITY) : ld4(xb + (long)(16 * q + 4 * t) * Cc);
        if constexpr (GRAD_A) xa[q & 1][t] = alrow[16 * q + 4 * t];
      }
    }
  };
  fetch(0);
  acc_rows(acc, reinterpret_cast<float*>(smem) + wave * kStripFloats, lane,
           [&](int q) __attribute__((always_inline)) { if (q + 1 < 4) fetch(q + 1); },
           [&](int q, int t, float4 v) __attribute__((always_inline)) {
             if (RAGGED && !(cok && 16 * q + 4 * t < rows_left)) return;
             float4 x;
             if constexpr (GRAD_A) x = exp4(xq[q & 1][t], xa[q & 1][t]);
             else x = exp4(xq[q & 1][t], becol);
             const float4 r = make_float4(x.x * v.x, x.y * v.y, x.z * v.z, x.w * v.w);
             if (RAGGED) st4m(gp + (long)(16 * q + 4 * t) * Cc, cc, r);
             else st4(gp + (long)(16 * q + 4 * t) * Cc, r);
           });
}

// Both gradients in one launch, item by item, a tile of each in turn (see k_log_bwd_mfma_both).
template <class TA, class TB, bool RAGGED>
__global__ __launch_bounds__(TA::NT) __attribute__((amdgpu_waves_per_eu(TA::WPE, TA::WPE)))
void k_log_bwd_split_both(const elem_t* __restrict__ g, const LeanSrc src, const int* __restrict__ ws_hdr,
                          const int* __restrict__ fwd_flags, elem_t* __restrict__ grad_a,
                          elem_t* __restrict__ grad_b, int M, int K, int N, int ar, int ac, int br, int bc) {
  static_assert(TA::NT == TB::NT && TA::WPE == TB::WPE, "");
  extern __shared__ __attribute__((aligned(16))) unsigned split_smem[];
  const int per_a = ar * ac, per_b = br * bc;
  const int v = xcd_renumber(blockIdx.x, gridDim.x);
  const int item = v / (per_a + per_b), r = v - item * (per_a + per_b);
  const bool alt = per_a == per_b;
  const bool is_a = alt ? (r & 1) == 0 : r < per_a;
  const int idx = alt ? r >> 1 : (r < per_a ? r : r - per_a);
  if (is_a)
    log_bwd_split_tile<TA, true, RAGGED>(split_smem, item * per_a + idx, g, src, ws_hdr, fwd_flags, grad_a, M, K, N, ar, ac);
  else
    log_bwd_split_tile<TB, false, RAGGED>(split_smem, item * per_b + idx, g, src, ws_hdr, fwd_flags, grad_b, M, K, N, br, bc);
}

template <class TA, class TB>
constexpr int split_bwd_lds_bytes() {
  constexpr int a = SplitBwd<TA, true>::WORDS, b = SplitBwd<TB, false>::WORDS;
  return 4 * (a > b ? a : b);
}

}  // namespace GENBMM_NS
