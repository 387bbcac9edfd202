// Factored logbmm on the fp32 matrix cores, for any sizes.  The loop has no bounds
// checks and no index arithmetic - each lane walks fixed pointers slab by slab -
// and ragged edges are dealt with outside it (see the RAGGED notes at the kernels).
//
// A workgroup of (TR/64) x (TC/64) waves owns a TR x TC output tile (128x128,
// 128x256 or 256x128); each wave keeps a 64x64 block as 2x2 accumulator blocks of
// v_mfma_f32_32x32x2_f32 (fp32 in, fp32 accumulate).  The reduction axis is
// consumed in slabs of 16 through two LDS buffers: while the matrix cores work on
// slab s, the global loads of slab s+1 are in flight; they are staged (forward:
// turned into exp(x - shift)) into the other buffer before the single barrier of
// the iteration.
#pragma once

#include "common.h"
#include "logbmm_ws.h"

namespace GENBMM_NS {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// D(32x32) += A(32x2) * B(2x32).  Lane l supplies A[l % 32][l / 32] and
// B[l / 32][l % 32] and holds D[8*(i/4) + 4*(l/32) + i%4][l % 32] in element i.
__device__ __forceinline__ floatx16 mfma_32x32x2(float a, float b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ int mfma_row(int i, int lane) {
  return 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
}
// The same split into a part that is uniform over the wave and the lane's part.
__device__ __forceinline__ constexpr int mfma_row_u(int i) { return 8 * (i >> 2) + (i & 3); }
__device__ __forceinline__ int mfma_row_l(int lane) { return 4 * (lane >> 5); }

constexpr int kMS = 16;         // slab depth
constexpr int kMPad = 4;        // LDS row padding (floats) of a [slab][tile] buffer
constexpr float kMfmaGuardBits = 40.f;

__device__ __forceinline__ int xcd_tile_id() { return xcd_renumber(blockIdx.x, gridDim.x); }

__device__ __forceinline__ float exp_st(float d) { return fast_exp2(d * kLog2e); }

// The matrix-core instruction runs on the same lanes as ordinary vector
// instructions (the hardware counters show no cycle of overlap), so every
// vector instruction spent on staging is taken from the contraction.  A tile is
// therefore TR x TC with one side 256 when the problem allows: each staged
// element then serves twice as many products, and the side whose staging is
// dearer (H in the backward kernels, the transposed stores elsewhere) is the
// short one.  (TR/64) x (TC/64) waves, each keeping a 64x64 block as 2x2
// accumulators of v_mfma_f32_32x32x2_f32.
template <int TR_, int TC_, int WPE_ = 4>
struct MTile {
  static constexpr int TR = TR_, TC = TC_;
  static constexpr int WPE = WPE_;              // waves per SIMD the kernel is compiled for
  static constexpr int WC = TC / 64;            // waves across
  static constexpr int NT = (TR / 64) * WC * 64;
  static constexpr int LDR = TR + kMPad, LDC = TC + kMPad;
};

// 32 matrix-core steps over one staged slab: rows from R[q][0..TR), columns
// from Cs[q][0..TC).
template <int LDR, int LDC>
__device__ __forceinline__ void mfma_slab(const float* __restrict__ R, const float* __restrict__ Cs,
                                          int wr0, int wc0, int lane, floatx16 (&acc)[2][2]) {
  const int lrow = lane & 31, lk = lane >> 5;
  const float* rp = R + lk * LDR + wr0 + lrow;
  const float* cp = Cs + lk * LDC + wc0 + lrow;
  // operands of step q+2 are read while the four products of step q run
  float fa[2][2], fb[2][2];
  __builtin_amdgcn_s_setprio(1);
  fa[0][0] = rp[0]; fa[0][1] = rp[32];
  fb[0][0] = cp[0]; fb[0][1] = cp[32];
  __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
  for (int q = 0; q < kMS; q += 2) {
    const int c = (q >> 1) & 1, n = c ^ 1;
    if (q + 2 < kMS) {
      fa[n][0] = rp[(q + 2) * LDR]; fa[n][1] = rp[(q + 2) * LDR + 32];
      fb[n][0] = cp[(q + 2) * LDC]; fb[n][1] = cp[(q + 2) * LDC + 32];
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    acc[0][0] = mfma_32x32x2(fa[c][0], fb[c][0], acc[0][0]);
    acc[0][1] = mfma_32x32x2(fa[c][0], fb[c][1], acc[0][1]);
    acc[1][0] = mfma_32x32x2(fa[c][1], fb[c][0], acc[1][0]);
    acc[1][1] = mfma_32x32x2(fa[c][1], fb[c][1], acc[1][1]);
    __builtin_amdgcn_sched_group_barrier(0x8, 4, 0);
  }
  __builtin_amdgcn_s_setprio(0);
}

// A staged operand tile of OUT lines x kMS reduction steps, one float4 per
// thread and piece.  Transposed: the source is [out][red] (float4 along red,
// four scalar LDS stores);  straight: the source is [red][out] (float4 along
// out, one 16-byte store).
template <int OUT, int NT, int LD>
struct StageT {
  static constexpr int PER = OUT * 4 / NT;
  static constexpr int STEP = NT / 4;  // source lines between a thread's pieces
  static_assert(PER >= 1 && OUT * 4 % NT == 0, "");
  static __device__ __forceinline__ int line(int tid, int l) { return (tid >> 2) + l * (NT / 4); }
  static __device__ __forceinline__ int quad(int tid) { return tid & 3; }
  // first reduction step (within the slab) of piece l; a piece spans four of them
  static __device__ __forceinline__ int redpos(int tid, int) { return (tid & 3) * 4; }
  static __device__ __forceinline__ void put(float* __restrict__ buf, int tid, int l, float4 v) {
    float* p = buf + (quad(tid) * 4) * LD + line(tid, l);
    p[0] = v.x; p[LD] = v.y; p[2 * LD] = v.z; p[3 * LD] = v.w;
  }
};
template <int OUT, int NT, int LD>
struct StageS {
  static constexpr int Q = OUT / 4;
  static constexpr int PER = kMS * Q / NT;
  static constexpr int STEP = NT / Q;  // source lines between a thread's pieces
  static_assert(PER >= 1 && kMS * Q % NT == 0 && NT % Q == 0, "");
  static __device__ __forceinline__ int red(int tid, int l) { return tid / Q + l * (NT / Q); }
  static __device__ __forceinline__ int quad(int tid) { return tid % Q; }
  // the reduction step (within the slab) of piece l
  static __device__ __forceinline__ int redpos(int tid, int l) { return red(tid, l); }
  static __device__ __forceinline__ void put(float* __restrict__ buf, int tid, int l, float4 v) {
    *reinterpret_cast<float4*>(buf + red(tid, l) * LD + quad(tid) * 4) = v;
  }
};

// Two arrays of the same shape - one of the caller's elements, one of fp32 workspace -
// are walked with one pointer: the element at the same index of the other array is
// found by integer arithmetic on addresses (not pointer arithmetic across objects).
// ws_twin: from an element pointer to the fp32 array; elem_twin: the other way round.
// The distance may carry a fixed offset in bytes of the target array.
template <class E>
constexpr uintptr_t kWiden = 4 / sizeof(E);  // bytes of workspace per byte of element
template <class E>
__device__ __forceinline__ long ws_distance(const float* ws, const E* from) {
  return (long)(reinterpret_cast<uintptr_t>(ws) - reinterpret_cast<uintptr_t>(from) * kWiden<E>);
}
// (The address is handed back through a pointer typed as global memory: a pointer made from a
// bare integer is of unknown address space, its accesses become flat_load / flat_store, and the
// compiler drains every outstanding global load before it issues one - the slab in flight
// under the matrix instructions would be waited for at the top of each step.)
template <class T>
using global_ptr = __attribute__((address_space(1))) T*;
template <class E>
__device__ __forceinline__ float* ws_twin(const E* p, long d) {
  return (float*)reinterpret_cast<global_ptr<float>>(reinterpret_cast<uintptr_t>(p) * kWiden<E> + (uintptr_t)d);
}
template <class E>
__device__ __forceinline__ long elem_distance(const E* to, const float* ws) {
  return (long)(reinterpret_cast<uintptr_t>(to) - reinterpret_cast<uintptr_t>(ws) / kWiden<E>);
}
template <class E>
__device__ __forceinline__ const E* elem_twin(const float* p, long d) {
  return (const E*)reinterpret_cast<global_ptr<const E>>(reinterpret_cast<uintptr_t>(p) / kWiden<E> + (uintptr_t)d);
}
__device__ __forceinline__ float4 exp4(float4 x, float4 s) {
  return make_float4(exp_st(x.x - s.x), exp_st(x.y - s.y), exp_st(x.z - s.z), exp_st(x.w - s.w));
}
__device__ __forceinline__ float4 exp4(float4 x, float s) {
  return make_float4(exp_st(x.x - s), exp_st(x.y - s), exp_st(x.z - s), exp_st(x.w - s));
}

// What the forward leaves in the caller's workspace for the backward kernels:
// EA = exp(a - alpha), EB = exp(b - beta) (each written by the tiles of the
// first column / row block while they stage them anyway) and R = 1/S per output
// cell, so that the backward contraction needs no exponential at all:
// H = g * R.  hdr[0] = 1 once they are valid, hdr[1], hdr[2] = the forward's
// tile shape (its flags tell which cells of R are not usable).  The kernels take
// the members as separate __restrict__ parameters: through a struct the
// compiler must assume that they alias the output and serialises the epilogue.
struct LogPrepared {
  float* ea;
  float* eb;
  float* r;
  int* hdr;
};

// Must a backward tile be left to the exact routine?  Yes if the workspace does not
// hold what the tile's kernel reads (need_factors: EA, EB, 1/S of the matrix-core
// forward; otherwise the flags of any factored forward), or if the forward flagged a
// tile among the cells this tile reduces over - rows [lo, lo + extent) of out and
// every column (by_rows: a grad_a tile), or columns [lo, lo + extent) and every row (a
// grad_b tile).  A pure function of what the forward left, so the backward kernel and
// its fix-up launch derive the same answer and nothing is written to the workspace.
// Every thread of the workgroup must call it (one barrier inside).
__device__ __forceinline__ int bwd_tile_flagged(const int* __restrict__ hdr,
                                                const int* __restrict__ fwd_flags,
                                                bool need_factors, bool by_rows, int lo, int extent,
                                                int batch, int M, int N, int tid, int nt) {
  const int tag = hdr[0], ftr = hdr[1], ftc = hdr[2];
  // flag words exist per 32 x 32 cells at the densest
  int bad = !(need_factors ? tag == kWsMfma : (tag == kWsMfma || tag == kWsFast)) || ftr < 32 || ftc < 32;
  if (!bad) {
    const int fm = (M + ftr - 1) / ftr, fn = (N + ftc - 1) / ftc;
    const int mlo = by_rows ? lo / ftr : 0, mhi = by_rows ? min((lo + extent - 1) / ftr, fm - 1) : fm - 1;
    const int nlo = by_rows ? 0 : lo / ftc, nhi = by_rows ? fn - 1 : min((lo + extent - 1) / ftc, fn - 1);
    const int nn = nhi - nlo + 1, cnt = (mhi - mlo + 1) * nn;
    for (int t = tid; t < cnt; t += nt)
      bad |= fwd_flags[((long)batch * fm + mlo + t / nn) * fn + nlo + t % nn];
  }
  return __syncthreads_or(bad);
}

// Compiler-level ordering point for a wave's own LDS traffic (the hardware
// executes one wave's LDS instructions in order).
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

constexpr int kStripFloats = 16 * 64;  // per wave: 16 rows of its 64-column block

// Hands a wave's 64x64 accumulator block back in row-major order, so that global
// memory is touched 16 bytes per lane and 256 contiguous bytes per row instead
// of 4 and 128: f(q, t, v) receives, for quarter q = 0..3 and t = 0..3, the four
// consecutive columns (lane & 15) * 4 .. +3 of block row 16*q + 4*t + (lane >> 4).
// `pre(q)` runs before quarter q is exchanged (a place to start loads).  The
// exchange goes through a wave-private LDS strip; the caller guarantees that no
// wave still reads the staging buffers the strip overlays.
template <class P, class F>
__device__ __forceinline__ void acc_rows(const floatx16 (&acc)[2][2], float* __restrict__ strip,
                                         int lane, P&& pre, F&& f) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    pre(q);
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int i = 0; i < 8; ++i)
        strip[(mfma_row_u(i) + mfma_row_l(lane)) * 64 + c * 32 + (lane & 31)] =
            acc[q >> 1][c][(q & 1) * 8 + i];
    wave_lds_sync();
    float4 v[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
      v[t] = *reinterpret_cast<const float4*>(strip + ((lane >> 4) + 4 * t) * 64 + (lane & 15) * 4);
    wave_lds_sync();
#pragma unroll
    for (int t = 0; t < 4; ++t) f(q, t, v[t]);
  }
}

// ----------------------------------------------------------------- forward
// rows <- EA from a[m][k] (transposed stage), columns <- EB from b[k][n].
//
// RAGGED: M, N need not be multiples of the tile nor K of the slab - any sizes.
// Lines of a tile beyond the matrix re-read the last line and get the shift +inf,
// i.e. exp -> 0, at no cost in the loop; a piece of four that straddles the right
// edge is read element by element by the few lanes that own one; the reduction
// tail is filled with -inf (exp -> 0) by a loader used for the last slab only;
// results and by-products are stored under masks.  Full-tile problems compile
// without any of it.
// KEEP: leave EA, EB and 1/S in the workspace for the backward (false: a forward
// for its own sake - the workspace then holds the maxima, flags and header only).
template <class T, bool RAGGED, bool KEEP = true>
__global__ __launch_bounds__(T::NT) __attribute__((amdgpu_waves_per_eu(T::WPE, T::WPE)))
void k_log_fwd_mfma(const elem_t* __restrict__ a, const elem_t* __restrict__ b,
                    elem_t* __restrict__ out, const float* __restrict__ stats,
                    int* __restrict__ flags, float* __restrict__ ws_ea,
                    float* __restrict__ ws_eb, float* __restrict__ ws_r, int* __restrict__ ws_hdr,
                    int M, int K, int N, int tiles_m, int tiles_n) {
  constexpr int NT = T::NT, LDR = T::LDR, LDC = T::LDC;
  using SA = StageT<T::TR, NT, LDR>;
  using SB = StageS<T::TC, NT, LDC>;
  __shared__ __attribute__((aligned(16))) float smem[2 * kMS * (LDR + LDC)];
  static_assert(2 * kMS * (LDR + LDC) >= (NT / 64) * kStripFloats, "");
  float(*As)[kMS * LDR] = reinterpret_cast<float(*)[kMS * LDR]>(smem);
  float(*Bs)[kMS * LDC] = reinterpret_cast<float(*)[kMS * LDC]>(smem + 2 * kMS * LDR);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps tile offsets scalar
  const int wm0 = (wave / T::WC) * 64, wn0 = (wave % T::WC) * 64;
  const int per = tiles_m * tiles_n, tile = xcd_tile_id();
  const int batch = tile / per, rem = tile - batch * per;
  const int m0 = (rem / tiles_n) * T::TR, n0 = (rem % tiles_n) * T::TC;
  const float* st = stats + (long)batch * (M + N);
  // EA / EB are written out by the tiles that stage them anyway: the tiles of
  // one row block share the slabs of EA between them (slab s goes to column
  // block s mod tiles_n), likewise EB, so that every workgroup stores the same.
  const int nblk = rem % tiles_n, mblk = rem / tiles_n;

  // a pieces: lines m0 + line(l), four k from quad*4;  b pieces: rows red(l), four n
  const int bcol = n0 + SB::quad(tid) * 4;
  const int cb = RAGGED ? clamp4(N - bcol) : 4;  // columns of this lane's b pieces inside the matrix
  const bool vb = cb > 0;
  bool va[SA::PER];
  const elem_t* pa[SA::PER];
  const elem_t* pb[SB::PER];
  float al[SA::PER];
#pragma unroll
  for (int l = 0; l < SA::PER; ++l) {
    const int line = m0 + SA::line(tid, l);
    va[l] = !RAGGED || line < M;
    pa[l] = a + ((long)batch * M + (va[l] ? line : M - 1)) * K + SA::quad(tid) * 4;
    al[l] = va[l] ? st[line] : INFINITY;
  }
#pragma unroll
  for (int l = 0; l < SB::PER; ++l)
    pb[l] = b + ((long)batch * K + SB::red(tid, l)) * N + (vb ? bcol : 0);
  const float4 be = RAGGED ? ld4m(st + M + (vb ? bcol : 0), cb, INFINITY) : ld4(st + M + bcol);
  // by-products live at the same offsets in their own arrays
  // (the source pointers run one slab ahead of what is being staged)
  const long da = ws_distance(ws_ea, a) - 4l * kMS, db = ws_distance(ws_eb, b) - 4l * kMS * N;
  if (tile == 0 && tid == 0) {
    ws_hdr[1] = T::TR;
    ws_hdr[2] = T::TC;
    ws_hdr[0] = KEEP ? kWsMfma : kWsFast;
  }

  floatx16 acc[2][2];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[x >> 1][x & 1][i] = 0.f;

  const int ktail = RAGGED ? K % kMS : 0;          // reduction steps of a partial last slab
  const int slabs = RAGGED ? (K + kMS - 1) / kMS : K / kMS;
  const float4 ninf = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
  float4 ra[SA::PER], rb[SB::PER];
  int ca = 4;                                      // reduction steps of the a pieces inside K
  bool tb[SB::PER];                                // b pieces inside K
#pragma unroll
  for (int l = 0; l < SB::PER; ++l) tb[l] = true;
  auto load = [&](bool tail) __attribute__((always_inline)) {
    if (RAGGED && tail) {
      ca = clamp4(ktail - SA::quad(tid) * 4);
#pragma unroll
      for (int l = 0; l < SA::PER; ++l) ra[l] = ld4m(pa[l], ca, -INFINITY);
#pragma unroll
      for (int l = 0; l < SB::PER; ++l) {
        tb[l] = SB::red(tid, l) < ktail;
        rb[l] = tb[l] ? ld4m(pb[l], cb, -INFINITY) : ninf;
      }
    } else {
#pragma unroll
      for (int l = 0; l < SA::PER; ++l) ra[l] = ld4(pa[l]);
#pragma unroll
      for (int l = 0; l < SB::PER; ++l) rb[l] = RAGGED ? ld4m(pb[l], cb, -INFINITY) : ld4(pb[l]);
    }
#pragma unroll
    for (int l = 0; l < SA::PER; ++l) pa[l] += kMS;
#pragma unroll
    for (int l = 0; l < SB::PER; ++l) pb[l] += (long)kMS * N;
  };
  auto stage = [&](int buf, bool keep_a, bool keep_b) __attribute__((always_inline)) {
#pragma unroll
    for (int l = 0; l < SA::PER; ++l) {
      const float4 e = exp4(ra[l], al[l]);
      SA::put(As[buf], tid, l, e);
      if (keep_a) {
        if (!RAGGED) st4(ws_twin(pa[l], da), e);
        else if (va[l]) st4m(ws_twin(pa[l], da), ca, e);
      }
    }
#pragma unroll
    for (int l = 0; l < SB::PER; ++l) {
      const float4 e = exp4(rb[l], be);
      SB::put(Bs[buf], tid, l, e);
      if (keep_b) {
        if (!RAGGED) st4(ws_twin(pb[l], db), e);
        else if (tb[l]) st4m(ws_twin(pb[l], db), cb, e);
      }
    }
  };

  load(slabs == 1 && ktail != 0);
  stage(0, KEEP && nblk == 0, KEEP && mblk == 0);
  __syncthreads();
  int sa = 1 % tiles_n, sb = 1 % tiles_m;  // (s + 1) mod tiles_n, mod tiles_m
  for (int s = 0; s < slabs; ++s) {
    const bool more = s + 1 < slabs;
    if (more) load(s + 2 == slabs && ktail != 0);
    mfma_slab<LDR, LDC>(As[s & 1], Bs[s & 1], wm0, wn0, lane, acc);
    if (more) stage((s + 1) & 1, KEEP && sa == nblk, KEEP && sb == mblk);
    sa = sa + 1 == tiles_n ? 0 : sa + 1;
    sb = sb + 1 == tiles_m ? 0 : sb + 1;
    __syncthreads();
  }

  // guard: S >= 2^-40 and finite; ...
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
  // ... every shift finite and not below the floor; and, since the reference keeps its running
  // maximum at the floor or above, alpha + beta of every cell within reach of the floor must not
  // be so far below it that the reference's terms would vanish (they do from 104 below): a row
  // at the floor (an operand row masked with -1e9) is factored as long as every column's shift
  // is above -30, and the other way round.  (1 / S is kept as computed, not derived from `out`,
  // so the backward loses nothing to the rounding of results near -1e9.)
  static_assert(T::TR + T::TC <= NT, "one shift per thread");
  int low = 0, neg = 0;  // bit 0: of a row, bit 1: of a column
  {
    const int t = tid;
    const bool row = t < T::TR;
    const bool here = t < T::TR + T::TC && (!RAGGED || (row ? m0 + t < M : n0 + t - T::TR < N));
    if (here) {
      const float sh = row ? st[m0 + t] : st[M + n0 + t - T::TR];
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

  // out = log S + alpha + beta and R = 1/S, written row-wise
  const int lr = lane >> 4, lc = (lane & 15) * 4;
  const int cc = RAGGED ? clamp4(N - (n0 + wn0 + lc)) : 4;  // columns of this lane's pieces that exist
  const bool cok = cc > 0;
  const float4 be4 = RAGGED ? ld4m(st + M + (cok ? n0 + wn0 + lc : 0), cc, 0.f) : ld4(st + M + n0 + wn0 + lc);
  const float* alw = st + m0 + wm0 + lr;
  const long ubase = ((long)batch * M + m0 + wm0) * N + n0 + wn0;
  const int voff = lr * N + lc;
  const int rows_left = M - (m0 + wm0) - lr;
  acc_rows(acc, smem + wave * kStripFloats, lane, [](int) {},
           [&](int q, int t, float4 sv) __attribute__((always_inline)) {
             const int ru = 16 * q + 4 * t;
             if (RAGGED && !(cok && ru < rows_left)) return;
             const float alr = alw[ru];
             const long u = ubase + (long)ru * N;
             const float4 rv = make_float4(__builtin_amdgcn_rcpf(sv.x), __builtin_amdgcn_rcpf(sv.y),
                                           __builtin_amdgcn_rcpf(sv.z), __builtin_amdgcn_rcpf(sv.w));
             const float4 ov = make_float4(__builtin_fmaf(fast_log2(sv.x), kLn2, alr + be4.x),
                                           __builtin_fmaf(fast_log2(sv.y), kLn2, alr + be4.y),
                                           __builtin_fmaf(fast_log2(sv.z), kLn2, alr + be4.z),
                                           __builtin_fmaf(fast_log2(sv.w), kLn2, alr + be4.w));
             if (RAGGED) {
               if (KEEP) st4m(ws_r + u + voff, cc, rv);
               st4m(out + u + voff, cc, ov);
             } else {
               if (KEEP) st4(ws_r + u + voff, rv);
               st4(out + u + voff, ov);
             }
           });
}

// ---------------------------------------------------------------- backward
// On the forward's by-products:  H = g * R.
// GRAD_A: tile (m,k) of grad_a = EA * sum_n H[m][n] EB[k][n]; rows <- H, columns
//         <- EB, both sources [out][red] (transposed stage).
// GRAD_B: tile (k,n) of grad_b = EB * sum_m EA[m][k] H[m][n]; rows <- EA,
//         columns <- H, both sources [red][out].
// A tile that touches a cell the forward flagged (R unusable there), or runs
// on a workspace the matrix-core forward did not fill, leaves its work to the
// fix-up launch, which finds it by the same test (bwd_tile_flagged).
// RAGGED (any sizes): lines of a tile beyond the matrix re-read the last line (they
// only feed results that are not stored); pieces straddling the right edge are
// read element by element; the reduction tail is zero-filled in both operands by
// the loader of the last slab; the epilogue is masked.
template <class T, bool GRAD_A, bool RAGGED>
__device__ __forceinline__ void log_bwd_mfma_tile(
    float* __restrict__ smem, int tile, const elem_t* __restrict__ g,
    const float* __restrict__ ws_ea, const float* __restrict__ ws_eb,
    const float* __restrict__ ws_r, const int* __restrict__ ws_hdr,
    const int* __restrict__ fwd_flags, elem_t* __restrict__ grad, int M, int K, int N, int tiles_r,
    int tiles_c) {
  constexpr int NT = T::NT, LDR = T::LDR, LDC = T::LDC;
  using SH = std::conditional_t<GRAD_A, StageT<T::TR, NT, LDR>, StageS<T::TC, NT, LDC>>;
  using SY = std::conditional_t<GRAD_A, StageT<T::TC, NT, LDC>, StageS<T::TR, NT, LDR>>;
  static_assert(2 * kMS * (LDR + LDC) >= (NT / 64) * kStripFloats, "");
  float(*Rs)[kMS * LDR] = reinterpret_cast<float(*)[kMS * LDR]>(smem);
  float(*Cs)[kMS * LDC] = reinterpret_cast<float(*)[kMS * LDC]>(smem + 2 * kMS * LDR);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps tile offsets scalar
  const int wr0 = (wave / T::WC) * 64, wc0 = (wave % T::WC) * 64;
  const int per = tiles_r * tiles_c;
  const int batch = tile / per, rem = tile - batch * per;
  const int r0 = (rem / tiles_c) * T::TR, c0 = (rem % tiles_c) * T::TC;
  const int Q = GRAD_A ? N : M;                      // reduction extent
  const int R = GRAD_A ? M : K, Cc = GRAD_A ? K : N;  // output extents

  floatx16 acc[2][2];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[x >> 1][x & 1][i] = 0.f;

  float4 ry[SY::PER], rr[SH::PER], rg[SH::PER];
  const float* py[SY::PER];
  const float* pr[SH::PER];
  long dg;  // g sits at the same element offsets as R
  // elements of this lane's pieces inside the matrix: grad_b pieces run along the
  // output axis (fixed per lane), grad_a pieces along the reduction (last slab only)
  int cy = 4, ch = 4;
  if constexpr (GRAD_A) {
#pragma unroll
    for (int l = 0; l < SY::PER; ++l) {  // EB[k][n]: line k, four n from quad*4
      const int k = c0 + SY::line(tid, l);
      py[l] = ws_eb + ((long)batch * K + (RAGGED ? min(k, K - 1) : k)) * N + SY::quad(tid) * 4;
    }
#pragma unroll
    for (int l = 0; l < SH::PER; ++l) {
      const int m = r0 + SH::line(tid, l);
      pr[l] = ws_r + ((long)batch * M + (RAGGED ? min(m, M - 1) : m)) * N + SH::quad(tid) * 4;
    }
  } else {
    const int kc = r0 + SY::quad(tid) * 4, nc = c0 + SH::quad(tid) * 4;
    cy = RAGGED ? clamp4(K - kc) : 4;
    ch = RAGGED ? clamp4(N - nc) : 4;
#pragma unroll
    for (int l = 0; l < SY::PER; ++l)    // EA[m][k]: row m = red, four k
      py[l] = ws_ea + ((long)batch * M + SY::red(tid, l)) * K + (cy > 0 ? kc : 0);
#pragma unroll
    for (int l = 0; l < SH::PER; ++l)
      pr[l] = ws_r + ((long)batch * M + SH::red(tid, l)) * N + (ch > 0 ? nc : 0);
  }
  dg = elem_distance(g, ws_r);
  const int qtail = RAGGED ? Q % kMS : 0;
  const int slabs = RAGGED ? (Q + kMS - 1) / kMS : Q / kMS;
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
  auto load = [&](bool tail) __attribute__((always_inline)) {
    if (!RAGGED) {
#pragma unroll
      for (int l = 0; l < SY::PER; ++l) ry[l] = ld4(py[l]);
#pragma unroll
      for (int l = 0; l < SH::PER; ++l) {
        rr[l] = ld4(pr[l]);
        rg[l] = ld4(elem_twin<elem_t>(pr[l], dg));
      }
    } else {
      // grad_a: a piece covers reduction steps redpos .. redpos+3; grad_b: one step
#pragma unroll
      for (int l = 0; l < SY::PER; ++l) {
        const int left = tail ? qtail - SY::redpos(tid, l) : 4;
        ry[l] = ld4m(py[l], GRAD_A ? left : (left > 0 ? cy : 0), 0.f);
      }
#pragma unroll
      for (int l = 0; l < SH::PER; ++l) {
        const int left = tail ? qtail - SH::redpos(tid, l) : 4;
        const int cnt = GRAD_A ? left : (left > 0 ? ch : 0);
        rr[l] = ld4m(pr[l], cnt, 0.f);
        rg[l] = ld4m(elem_twin<elem_t>(pr[l], dg), cnt, 0.f);
      }
    }
#pragma unroll
    for (int l = 0; l < SY::PER; ++l) py[l] += GRAD_A ? (long)kMS : (long)kMS * K;
#pragma unroll
    for (int l = 0; l < SH::PER; ++l) pr[l] += GRAD_A ? (long)kMS : (long)kMS * N;
  };
  auto stage = [&](int buf) __attribute__((always_inline)) {
    float* ybuf = GRAD_A ? Cs[buf] : Rs[buf];
    float* hbuf = GRAD_A ? Rs[buf] : Cs[buf];
#pragma unroll
    for (int l = 0; l < SY::PER; ++l) SY::put(ybuf, tid, l, ry[l]);
#pragma unroll
    for (int l = 0; l < SH::PER; ++l)
      SH::put(hbuf, tid, l, make_float4(rg[l].x * rr[l].x, rg[l].y * rr[l].y, rg[l].z * rr[l].z,
                                        rg[l].w * rr[l].w));
  };

  load(slabs == 1 && qtail != 0);
  // Forward flags over the cells this tile reduces over: the fix-up launch takes a flagged tile.
  // Asked while the first slab's loads are in flight (the workspace is allocated whatever it
  // holds, so the loads are harmless for a tile that then leaves).
  if (bwd_tile_flagged(ws_hdr, fwd_flags, true, GRAD_A, GRAD_A ? r0 : c0, GRAD_A ? T::TR : T::TC, batch,
                       M, N, tid, NT))
    return;
  stage(0);
  __syncthreads();
  for (int s = 0; s < slabs; ++s) {
    const bool more = s + 1 < slabs;
    if (more) load(s + 2 == slabs && qtail != 0);
    mfma_slab<LDR, LDC>(Rs[s & 1], Cs[s & 1], wr0, wc0, lane, acc);
    if (more) stage((s + 1) & 1);
    __syncthreads();
  }

  // grad = EX * acc, EX = EA or EB, row-wise; the loads of a quarter are started
  // before the previous quarter is exchanged.
  const int lr = lane >> 4, lc = (lane & 15) * 4;
  const int voff = lr * Cc + lc;
  const long ubase = ((long)batch * R + r0 + wr0) * Cc + c0 + wc0;
  const float* xb = (GRAD_A ? ws_ea : ws_eb) + ubase + voff;
  elem_t* gp = grad + ubase + voff;
  const int cc = RAGGED ? clamp4(Cc - (c0 + wc0 + lc)) : 4;  // columns of this lane's pieces that exist
  const bool cok = cc > 0;
  const int rows_left = R - (r0 + wr0) - lr;
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
             if (RAGGED && !(cok && 16 * q + 4 * t < rows_left)) return;
             const float4 x = xq[q & 1][t];
             const float4 r = make_float4(x.x * v.x, x.y * v.y, x.z * v.z, x.w * v.w);
             if (RAGGED) st4m(gp + (long)(16 * q + 4 * t) * Cc, cc, r);
             else st4(gp + (long)(16 * q + 4 * t) * Cc, r);
           });
}

template <class T, bool GRAD_A, bool RAGGED>
__global__ __launch_bounds__(T::NT) __attribute__((amdgpu_waves_per_eu(T::WPE, T::WPE)))
void k_log_bwd_mfma(const elem_t* __restrict__ g, const float* __restrict__ ws_ea,
                    const float* __restrict__ ws_eb, const float* __restrict__ ws_r,
                    const int* __restrict__ ws_hdr, const int* __restrict__ fwd_flags,
                    elem_t* __restrict__ grad, int M, int K, int N, int tiles_r, int tiles_c) {
  __shared__ __attribute__((aligned(16))) float smem[2 * kMS * (T::LDR + T::LDC)];
  log_bwd_mfma_tile<T, GRAD_A, RAGGED>(smem, xcd_tile_id(), g, ws_ea, ws_eb, ws_r, ws_hdr, fwd_flags,
                                       grad, M, K, N, tiles_r, tiles_c);
}

// Both gradients in one launch: the tiles of grad_a (shape TA) and of grad_b (shape TB),
// tiles_a of the former in all.
template <class TA, class TB, bool RAGGED>
__global__ __launch_bounds__(TA::NT) __attribute__((amdgpu_waves_per_eu(TA::WPE, TA::WPE)))
void k_log_bwd_mfma_both(const elem_t* __restrict__ g, const float* __restrict__ ws_ea,
                         const float* __restrict__ ws_eb, const float* __restrict__ ws_r,
                         const int* __restrict__ ws_hdr, const int* __restrict__ fwd_flags,
                         elem_t* __restrict__ grad_a, elem_t* __restrict__ grad_b, int M, int K, int N,
                         int tiles_a, int ar, int ac, int br, int bc) {
  static_assert(TA::NT == TB::NT && TA::WPE == TB::WPE, "");
  constexpr int kA = 2 * kMS * (TA::LDR + TA::LDC), kB = 2 * kMS * (TB::LDR + TB::LDC);
  __shared__ __attribute__((aligned(16))) float smem[kA > kB ? kA : kB];
  // Item by item, the tiles of grad_a and those of grad_b: both gradients of an item read the
  // same four arrays (g, 1/S, EA, EB: one's operand is the other's epilogue factor), so with
  // an item's tiles in flight together the second use of each comes from the XCD's L2
  // (all grad_a tiles first, then all grad_b tiles: 0.3125 against 0.3015 ms at the headline
  // shape, build against build on one box).  XCD-aware numbering over the whole launch.
  const int w = blockIdx.x, n = gridDim.x;
  const int per_a = ar * ac, per_b = br * bc;
  const int v = xcd_renumber(w, n);
  const int item = v / (per_a + per_b), r = v - item * (per_a + per_b);
  // (one of each in turn where an item has as many of either: another 0.4 %)
  const bool alt = per_a == per_b;
  const bool is_a = alt ? (r & 1) == 0 : r < per_a;
  const int idx = alt ? r >> 1 : (r < per_a ? r : r - per_a);
  if (is_a)
    log_bwd_mfma_tile<TA, true, RAGGED>(smem, item * per_a + idx, g, ws_ea, ws_eb, ws_r, ws_hdr, fwd_flags,
                                        grad_a, M, K, N, ar, ac);
  else
    log_bwd_mfma_tile<TB, false, RAGGED>(smem, item * per_b + idx, g, ws_ea, ws_eb, ws_r, ws_hdr,
                                         fwd_flags, grad_b, M, K, N, br, bc);
}

// ------------------------------------------------- backward without by-products
// The same two contractions for a forward that kept nothing but the maxima and its flags (a
// workspace of B (M + N) floats and a flag per tile instead of EA, EB and 1/S: at 64 x 512^3,
// 0.3 MB instead of 201 MB): the operands are formed again while they are staged -
// EA = exp(a - alpha), EB = exp(b - beta), H = g exp(alpha + beta - out) - and so is the
// epilogue's factor: exponentials per staged element where the kernels above multiply once.
// Shifts: alpha[m] of a piece's line (grad_a) or reduction step (grad_b), beta[n] of its four
// columns.  RAGGED as above, with fills that make the exponential vanish: -inf for a and b,
// +inf for out, 0 for g.
struct LeanSrc {
  const elem_t* a;
  const elem_t* b;
  const elem_t* out;
  const float* stats;  // alpha (M) then beta (N) per batch item
};
__device__ __forceinline__ float4 mul_exp4(float4 g, float4 sh, float4 o) {  // g * exp(sh - o)
  return make_float4(g.x * exp_st(sh.x - o.x), g.y * exp_st(sh.y - o.y), g.z * exp_st(sh.z - o.z),
                     g.w * exp_st(sh.w - o.w));
}
template <class T, bool GRAD_A, bool RAGGED>
__device__ __forceinline__ void log_bwd_mfma_tile_lean(
    float* __restrict__ smem, int tile, const elem_t* __restrict__ g, const LeanSrc src,
    const int* __restrict__ ws_hdr, const int* __restrict__ fwd_flags, elem_t* __restrict__ grad,
    int M, int K, int N, int tiles_r, int tiles_c) {
  constexpr int NT = T::NT, LDR = T::LDR, LDC = T::LDC;
  using SH = std::conditional_t<GRAD_A, StageT<T::TR, NT, LDR>, StageS<T::TC, NT, LDC>>;
  using SY = std::conditional_t<GRAD_A, StageT<T::TC, NT, LDC>, StageS<T::TR, NT, LDR>>;
  float(*Rs)[kMS * LDR] = reinterpret_cast<float(*)[kMS * LDR]>(smem);
  float(*Cs)[kMS * LDC] = reinterpret_cast<float(*)[kMS * LDC]>(smem + 2 * kMS * LDR);
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

  float4 ry[SY::PER], ro[SH::PER], rg[SH::PER];
  const elem_t* py[SY::PER];
  const elem_t* po[SH::PER];
  // g sits at the same element offsets as out (address arithmetic on integers, the result typed
  // as global memory: see ws_twin)
  const long dg = (long)(reinterpret_cast<uintptr_t>(g) - reinterpret_cast<uintptr_t>(src.out));
  auto g_of = [&](const elem_t* o) __attribute__((always_inline)) {
    return (const elem_t*)reinterpret_cast<global_ptr<const elem_t>>(reinterpret_cast<uintptr_t>(o) + (uintptr_t)dg);
  };
  // shifts.  grad_a: alpha of the H pieces' lines (fixed), beta of the slab's four columns (one
  // float4 per slab, the same for every piece: all pieces of a thread share their quad).
  // grad_b: beta of the lane's four columns (fixed), alpha of every piece's reduction step.
  float alh[SH::PER];
  const float* pbe = be + SH::quad(tid) * 4;  // grad_a: + kMS per slab
  float4 be4 = make_float4(0.f, 0.f, 0.f, 0.f), bslab = be4;
  float ay[SY::PER], ah[SH::PER];
  int cy = 4, ch = 4;
  if constexpr (GRAD_A) {
#pragma unroll
    for (int l = 0; l < SY::PER; ++l) {  // b[k][n]: line k, four n from quad*4
      const int k = c0 + SY::line(tid, l);
      py[l] = src.b + ((long)batch * K + (RAGGED ? min(k, K - 1) : k)) * N + SY::quad(tid) * 4;
    }
#pragma unroll
    for (int l = 0; l < SH::PER; ++l) {
      const int m = r0 + SH::line(tid, l);
      const int mc = RAGGED ? min(m, M - 1) : m;
      po[l] = src.out + ((long)batch * M + mc) * N + SH::quad(tid) * 4;
      alh[l] = al[mc];
    }
  } else {
    const int kc = r0 + SY::quad(tid) * 4, nc = c0 + SH::quad(tid) * 4;
    cy = RAGGED ? clamp4(K - kc) : 4;
    ch = RAGGED ? clamp4(N - nc) : 4;
#pragma unroll
    for (int l = 0; l < SY::PER; ++l)    // a[m][k]: row m = red, four k
      py[l] = src.a + ((long)batch * M + SY::red(tid, l)) * K + (cy > 0 ? kc : 0);
#pragma unroll
    for (int l = 0; l < SH::PER; ++l)
      po[l] = src.out + ((long)batch * M + SH::red(tid, l)) * N + (ch > 0 ? nc : 0);
    be4 = RAGGED ? ld4m(be + (ch > 0 ? nc : 0), ch, 0.f) : ld4(be + nc);
  }
  const int qtail = RAGGED ? Q % kMS : 0;
  const int slabs = RAGGED ? (Q + kMS - 1) / kMS : Q / kMS;
  int s_load = 0;  // slab the next load() fetches
  auto load = [&](bool tail) __attribute__((always_inline)) {
    const int q0 = s_load * kMS;
    if constexpr (GRAD_A) {
      const int left = tail ? qtail - SH::redpos(tid, 0) : 4;  // all pieces share their quad
      if (!RAGGED) {
#pragma unroll
        for (int l = 0; l < SY::PER; ++l) ry[l] = ld4(py[l]);
#pragma unroll
        for (int l = 0; l < SH::PER; ++l) {
          ro[l] = ld4(po[l]);
          rg[l] = ld4(g_of(po[l]));
        }
        bslab = ld4(pbe);
      } else {
#pragma unroll
        for (int l = 0; l < SY::PER; ++l) ry[l] = ld4m(py[l], left, -INFINITY);
#pragma unroll
        for (int l = 0; l < SH::PER; ++l) {
          ro[l] = ld4m(po[l], left, INFINITY);
          rg[l] = ld4m(g_of(po[l]), left, 0.f);
        }
        bslab = ld4m(pbe, left, 0.f);
      }
      pbe += kMS;
    } else {
#pragma unroll
      for (int l = 0; l < SY::PER; ++l) {
        const bool in = !RAGGED || !tail || SY::redpos(tid, l) < qtail;
        ry[l] = RAGGED ? ld4m(py[l], in ? cy : 0, -INFINITY) : ld4(py[l]);
        ay[l] = in ? al[q0 + SY::red(tid, l)] : 0.f;
      }
#pragma unroll
      for (int l = 0; l < SH::PER; ++l) {
        const bool in = !RAGGED || !tail || SH::redpos(tid, l) < qtail;
        ro[l] = RAGGED ? ld4m(po[l], in ? ch : 0, INFINITY) : ld4(po[l]);
        rg[l] = RAGGED ? ld4m(g_of(po[l]), in ? ch : 0, 0.f) : ld4(g_of(po[l]));
        ah[l] = in ? al[q0 + SH::red(tid, l)] : 0.f;
      }
    }
#pragma unroll
    for (int l = 0; l < SY::PER; ++l) py[l] += GRAD_A ? (long)kMS : (long)kMS * K;
#pragma unroll
    for (int l = 0; l < SH::PER; ++l) po[l] += GRAD_A ? (long)kMS : (long)kMS * N;
    ++s_load;
  };
  auto stage = [&](int buf) __attribute__((always_inline)) {
    float* ybuf = GRAD_A ? Cs[buf] : Rs[buf];
    float* hbuf = GRAD_A ? Rs[buf] : Cs[buf];
#pragma unroll
    for (int l = 0; l < SY::PER; ++l) {
      if constexpr (GRAD_A) SY::put(ybuf, tid, l, exp4(ry[l], bslab));
      else SY::put(ybuf, tid, l, exp4(ry[l], ay[l]));
    }
#pragma unroll
    for (int l = 0; l < SH::PER; ++l) {
      float4 sh;
      if constexpr (GRAD_A) sh = make_float4(alh[l] + bslab.x, alh[l] + bslab.y, alh[l] + bslab.z, alh[l] + bslab.w);
      else sh = make_float4(ah[l] + be4.x, ah[l] + be4.y, ah[l] + be4.z, ah[l] + be4.w);
      SH::put(hbuf, tid, l, mul_exp4(rg[l], sh, ro[l]));
    }
  };

  load(slabs == 1 && qtail != 0);
  if (bwd_tile_flagged(ws_hdr, fwd_flags, false, GRAD_A, GRAD_A ? r0 : c0, GRAD_A ? T::TR : T::TC, batch,
                       M, N, tid, NT))
    return;
  stage(0);
  __syncthreads();
  for (int s = 0; s < slabs; ++s) {
    const bool more = s + 1 < slabs;
    if (more) load(s + 2 == slabs && qtail != 0);
    mfma_slab<LDR, LDC>(Rs[s & 1], Cs[s & 1], wr0, wc0, lane, acc);
    if (more) stage((s + 1) & 1);
    __syncthreads();
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
  acc_rows(acc, smem + wave * kStripFloats, lane,
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

template <class T, bool GRAD_A, bool RAGGED>
__global__ __launch_bounds__(T::NT) __attribute__((amdgpu_waves_per_eu(T::WPE, T::WPE)))
void k_log_bwd_mfma_lean(const elem_t* __restrict__ g, const LeanSrc src, const int* __restrict__ ws_hdr,
                         const int* __restrict__ fwd_flags, elem_t* __restrict__ grad, int M, int K, int N,
                         int tiles_r, int tiles_c) {
  __shared__ __attribute__((aligned(16))) float smem[2 * kMS * (T::LDR + T::LDC)];
  log_bwd_mfma_tile_lean<T, GRAD_A, RAGGED>(smem, xcd_tile_id(), g, src, ws_hdr, fwd_flags, grad, M, K, N, tiles_r,
                                            tiles_c);
}

// Both gradients in one launch, item by item (see k_log_bwd_mfma_both): here the two share
// a, b, out and g.
template <class TA, class TB, bool RAGGED>
__global__ __launch_bounds__(TA::NT) __attribute__((amdgpu_waves_per_eu(TA::WPE, TA::WPE)))
void k_log_bwd_mfma_both_lean(const elem_t* __restrict__ g, const LeanSrc src, const int* __restrict__ ws_hdr,
                              const int* __restrict__ fwd_flags, elem_t* __restrict__ grad_a,
                              elem_t* __restrict__ grad_b, int M, int K, int N, int tiles_a, int ar, int ac,
                              int br, int bc) {
  static_assert(TA::NT == TB::NT && TA::WPE == TB::WPE, "");
  constexpr int kA = 2 * kMS * (TA::LDR + TA::LDC), kB = 2 * kMS * (TB::LDR + TB::LDC);
  __shared__ __attribute__((aligned(16))) float smem[kA > kB ? kA : kB];
  const int per_a = ar * ac, per_b = br * bc;
  const int v = xcd_renumber(blockIdx.x, gridDim.x);
  const int item = v / (per_a + per_b), r = v - item * (per_a + per_b);
  const bool alt = per_a == per_b;
  const bool is_a = alt ? (r & 1) == 0 : r < per_a;
  const int idx = alt ? r >> 1 : (r < per_a ? r : r - per_a);
  if (is_a)
    log_bwd_mfma_tile_lean<TA, true, RAGGED>(smem, item * per_a + idx, g, src, ws_hdr, fwd_flags, grad_a, M, K, N, ar, ac);
  else
    log_bwd_mfma_tile_lean<TB, false, RAGGED>(smem, item * per_b + idx, g, src, ws_hdr, fwd_flags, grad_b, M, K, N, br, bc);
}

// ------------------------------------------------------- sampling sweep
// samplebmm on the forward's factors: index = first k whose prefix sum
// sum_{k' <= k} EA[m,k'] EB[k',n] passes the target t = u * S (one Philox uniform
// u per cell, S = the reciprocal of the forward's 1 / S).  The accumulators start at -t, so after
// every slab they hold prefix - t: negative while the prefix is below the target, and
// closer to zero slab by slab.  One register per cell keeps what is needed of that
// history: the low six bits of the value's bit pattern are replaced by 62 - slab and
// a signed-integer minimum is taken (negative floats order backwards as integers and
// lie below every non-negative one; of two slabs the later has the smaller magnitude
// and the smaller tag, so it always wins).  At the end the tag gives the number of
// slabs that ended below the target = the slab in which the prefix passes it, and the
// value (six mantissa bits short) is -(t - prefix at the start of that slab) = -rem.
// Two vector instructions per cell and slab beside the matrix-core work.  Results:
// the code -2 - slab in idx (K - 1, the final index, if the prefix never reaches t: the
// accumulators start at -t, so their roundings are not the forward's, and a draw within some
// 1e-6 of 1 can end a hair above the sum) and rem in `remw`; the
// terms of that one slab are walked by the resolve kernel.  At most kSampleSlabs
// slabs: up to 62 with a tag of six bits, beyond that with seven (rem is then seven mantissa
// bits short: 1.5e-5 of itself, which moves a boundary between two terms by at most that
// share of the cell's total mass).  A tile with a cell whose S is below 2^-40 or not finite,
// or that lies in a tile the forward flagged, sets that flag and leaves: the forward's
// tile is redone exactly.  The sweep's own tile shape is free: 128 x 128 with four
// waves lets two workgroups share a compute unit within the 256 registers per lane,
// so that one's vector work overlaps the other's matrix-core work.
constexpr int kSampleSlabs = 126;
// The reciprocal of the forward's 1 / S is S within two roundings; a target within 2^-22 of the sum
// the sweep adds up could lie beyond it and never be passed.  Every target is shrunk by that
// much instead (the boundaries between the terms move by 2.4e-7 of the total mass).
constexpr float kSampleShrink = 1.f - 0x1p-22f;

}  // namespace GENBMM_NS
