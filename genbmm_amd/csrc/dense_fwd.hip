// Dense semiring batched matmul, forward kernels (gfx950 / CDNA4, wave64).
//
//   out[b,m,n] = (+)_k  a[b,m,k] (x) b[b,k,n]
//
// for the log (logsumexp, +), max (max, +), prod-max (max, *) and sampling
// semirings of the reference (matmul_cuda_kernel.cu:13-152).  These are not
// (+,*) contractions, so everything runs on the vector ALU: a workgroup owns a
// BM x BN output tile, streams K in KT-wide slabs through LDS (A transposed to
// [k][m] so that both operands are read as broadcast / conflict-free float4
// fragments) and every lane keeps a TM x TN block of running states in
// registers.  Lanes run along n, so the reads of b and the writes of out/idx
// are coalesced (the reference puts threadIdx.x on rows and strides by K/N).
#include "dense_tiles.h"
#include "logbmm_ws.h"

namespace GENBMM_NS {
namespace {

// ------------------------------------------------------- max / prod-max forward
// Reference: max_cuda_forward_kernel (matmul_cuda_kernel.cu:47-75) and
// prod_max_cuda_forward_kernel (:124-152): ascending k, strict '>', running
// maximum starts at -1e9 with index -1.
//
// Two levels.  The sweep keeps, per cell, the running maximum and the number of
// the group of kMaxGroup consecutive k in which that maximum was last raised: per
// term one add (multiply) and half a three-operand maximum, per group one compare
// and one select, instead of a compare and two selects per term.  The group
// number is written as the code -2 - group (-1: nothing exceeded -1e9).
// k_max_resolve then recomputes the terms of that one group per cell and stores
// their maximum and the first k whose term equals it, which is what the
// reference's walk with a strict comparison keeps: a later group only takes over
// with a strictly larger term, and inside the group the first equal term is the
// one that raised the maximum.  A NaN term never wins, in the walk (NaN > m is
// false) as in v_max_f32.
constexpr int kMaxGroup = 8;

template <class C, bool PROD>
__global__ __launch_bounds__(C::NT) void k_max_fwd(const DenseArgs p) {
  __shared__ __attribute__((aligned(16))) float As[C::KT * C::LDA];
  __shared__ __attribute__((aligned(16))) float Bs[C::KT * C::LDB];
  static_assert(C::KT % kMaxGroup == 0 && kMaxGroup % 2 == 0, "whole groups per slab");
  const int tid = threadIdx.x, tx = tid % C::TX, ty = tid / C::TX;
  int batch, m0, n0;
  decode_tile<C>(p, batch, m0, n0);
  const int M = p.M, K = p.K, N = p.N;
  const elem_t* ab = p.a + (long)batch * M * K;
  const elem_t* bb = p.b + (long)batch * K * N;

  float mx[C::TM][C::TN];
  int ind[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
      mx[i][j] = kFloor;
      ind[i][j] = -1;
    }

  TileOutMajor<C::BM, C::KT, C::NT> ta;
  TileRedMajor<C::BN, C::KT, C::NT> tb;
  if (K > 0) {
    ta.gload(ab, K, m0, 0, M, K, p.vec_a, tid);
    tb.gload(bb, N, n0, 0, N, K, p.vec_b, tid);
  }
  for (int k0 = 0; k0 < K; k0 += C::KT) {
    __syncthreads();
    ta.sstore(As, tid);
    tb.sstore(Bs, tid);
    __syncthreads();
    if (k0 + C::KT < K) {
      ta.gload(ab, K, m0, k0 + C::KT, M, K, p.vec_a, tid);
      tb.gload(bb, N, n0, k0 + C::KT, N, K, p.vec_b, tid);
    }
    const int kn = min(C::KT, K - k0);
    auto two = [&](int kk) __attribute__((always_inline)) {
      float a0[C::TM], b0[C::TN], a1[C::TM], b1[C::TN];
      lds_frag<C::TM / 4>(As + kk * C::LDA, ty * C::TM, 4, a0);
      lds_frag<C::TN / 4>(Bs + kk * C::LDB, tx * 4, C::TX * 4, b0);
      lds_frag<C::TM / 4>(As + (kk + 1) * C::LDA, ty * C::TM, 4, a1);
      lds_frag<C::TN / 4>(Bs + (kk + 1) * C::LDB, tx * 4, C::TX * 4, b1);
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
          const float t0 = PROD ? a0[i] * b0[j] : a0[i] + b0[j];
          const float t1 = PROD ? a1[i] * b1[j] : a1[i] + b1[j];
          mx[i][j] = __builtin_fmaxf(__builtin_fmaxf(mx[i][j], t0), t1);
        }
    };
    auto one = [&](int kk) __attribute__((always_inline)) {
      float a0[C::TM], b0[C::TN];
      lds_frag<C::TM / 4>(As + kk * C::LDA, ty * C::TM, 4, a0);
      lds_frag<C::TN / 4>(Bs + kk * C::LDB, tx * 4, C::TX * 4, b0);
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
          mx[i][j] = __builtin_fmaxf(mx[i][j], PROD ? a0[i] * b0[j] : a0[i] + b0[j]);
    };
#pragma unroll
    for (int g = 0; g < C::KT / kMaxGroup; ++g) {
      const int kg = g * kMaxGroup;
      if (kg >= kn) break;
      float before[C::TM][C::TN];
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j) before[i][j] = mx[i][j];
      if (kg + kMaxGroup <= kn) {
#pragma unroll
        for (int kk = 0; kk < kMaxGroup; kk += 2) two(kg + kk);
      } else {
        for (int kk = kg; kk < kn; ++kk) one(kk);
      }
      const int code = -2 - (k0 / kMaxGroup + g);
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
          if (mx[i][j] > before[i][j]) ind[i][j] = code;
    }
  }
  // the values come with the indices from k_max_resolve; without terms there is none
  if (K == 0) store_tile_f<C>(p.out + (long)batch * M * N, mx, m0, n0, M, N, p.vec_o, tx, ty);
  store_tile_i<C>(p.idx + (long)batch * M * N, ind, m0, n0, M, N, p.vec_o, tx, ty);
}

// Second level (max / prod-max and the sampling sweep): group code -> result.
// A workgroup owns COLS columns of one batch item and a range of rows; the rows of
// the second operand that the groups can point at are staged in LDS as [k][column]
// - 64 KB: 256 rows of 64 columns or 512 rows of 32 - so that a lane reads the bank
// of its own column whatever k it needs (COLS = 32: a wave takes two rows at a time
// and the two halves may meet in a bank).  The kResGroup values of the first operand
// come from the row the lanes of a half-wave share.  Rows are taken kResRows at a time,
// software-pipelined: the codes two steps ahead and the first operand's values one step
// ahead are requested before the current rows are finished and stored.
//
// Op supplies what differs: Extra load(e) (read together with the code of cell e),
// none(e) (a cell whose code is -1) and cell(e, kb, av, br, stride, valid, extra) with
// av[j] = first operand at k = kb + j, br[j * stride] = second operand, valid = number
// of terms of the group that lie inside K.
constexpr int kResGroup = 8, kResWaves = 8, kResRows = 4, kResStage = 8;
constexpr int kResFloats = 16384;  // 64 KB of LDS
static_assert(kMaxGroup == kResGroup, "");

// E: element type of the two operands (the caller's for max / prod-max, fp32 for the
// factors the sampling sweep runs on).
template <int COLS, bool TAIL, int G, int R, class E, class Op>
__device__ __forceinline__ void resolve_walk(const E* __restrict__ first, const E* __restrict__ second,
                                             int32_t* __restrict__ idx, Op& op, int M, int K, int N,
                                             int panels, int row_chunks, int rows_per, float* Bs) {
  constexpr int RPW = 64 / COLS;           // rows a wave takes per step
  constexpr int KSTAGE = kResFloats / COLS;  // rows of the second operand staged at a time
  constexpr int STEP = kResWaves * R * RPW;
  static_assert(KSTAGE % G == 0 && G % 4 == 0, "a group lies in one staged chunk");
  const int lane = threadIdx.x & 63, col = lane % COLS, sub = lane / COLS;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // the panels of a batch item share its rows of the first operand: keep them on one XCD (one L2)
  int wg = xcd_renumber(blockIdx.x, gridDim.x);
  const int panel = wg % panels;
  wg /= panels;
  const int chunk = wg % row_chunks;
  const int batch = wg / row_chunks;
  const int n = panel * COLS + col;
  const bool live = n < N;
  const int nc = min(n, N - 1);
  const int m_beg = chunk * rows_per, m_end = min(M, m_beg + rows_per);
  const E* ab = first + (long)batch * M * K;
  const E* bb = second + (long)batch * K * N;
  const long cell0 = (long)batch * M * N;
  const int32_t* ib = idx + cell0;
  using Extra = typename Op::Extra;
  auto row_of = [&](int mb, int r) { return mb + r * RPW + sub; };

  // codes of R rows (0: nothing to do, also outside the matrix) and what Op reads with them
  auto load_codes = [&](int mb, int (&code)[R], Extra (&ex)[R]) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int m = row_of(mb, r);
      const long e = (long)min(m, M - 1) * N + nc;
      const int c = ib[e];
      ex[r] = op.load(cell0 + e);
      code[r] = (live && m < m_end) ? c : 0;
    }
  };
  // first k of each row's group (-1: not a group of the staged rows kc..) and the
  // group's values of the first operand
  auto gather = [&](int mb, int kc, const int (&code)[R], int (&kb)[R], float (&av)[R][G])
                    __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int k = (-2 - code[r]) * G;
      const bool act = code[r] <= -2 && k >= kc && k < kc + KSTAGE;
      kb[r] = act ? k : -1;
      const int ks = act ? k : kc;
      const E* ar = ab + (long)min(row_of(mb, r), M - 1) * K + ks;
      if (!TAIL) {
#pragma unroll
        for (int q = 0; q < G / 4; ++q) {
          const float4 x = ld4(ar + 4 * q);
          av[r][4 * q] = x.x; av[r][4 * q + 1] = x.y; av[r][4 * q + 2] = x.z; av[r][4 * q + 3] = x.w;
        }
      } else {
#pragma unroll
        for (int j = 0; j < G; ++j) av[r][j] = ar[min(j, K - 1 - ks)];
      }
    }
  };
  auto finish = [&](int mb, int kc, int rows, const int (&code)[R], const Extra (&ex)[R],
                    const int (&kb)[R], const float (&av)[R][G]) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const long e = cell0 + (long)row_of(mb, r) * N + n;
      if (code[r] == -1 && kc == 0) op.none(e);
      if (kb[r] < 0) continue;
      const int rel = kb[r] - kc;
      // the last group of a ragged K: its rows past K are not staged; point at row rows - 1
      const float* br = Bs + rel * COLS + col;
      const int valid = TAIL ? min(G, K - kb[r]) : G;
      op.cell(e, kb[r], av[r], br, COLS, valid, min(G, rows - rel), ex[r]);
    }
  };

  for (int kc = 0; kc < K; kc += KSTAGE) {
    const int rows = min(KSTAGE, K - kc);
    int mb = m_beg + wave * R * RPW;
    int c0[R], c1[R], kb0[R];
    Extra e0[R], e1[R];
    float a0[R][G];
    load_codes(mb, c0, e0);
    __syncthreads();
    for (int r0 = wave * RPW + sub; r0 < rows; r0 += kResWaves * RPW * kResStage) {
      float x[kResStage];
#pragma unroll
      for (int u = 0; u < kResStage; ++u)
        x[u] = bb[(long)(kc + min(r0 + u * kResWaves * RPW, rows - 1)) * N + nc];
#pragma unroll
      for (int u = 0; u < kResStage; ++u)
        if (r0 + u * kResWaves * RPW < rows) Bs[(r0 + u * kResWaves * RPW) * COLS + col] = x[u];
    }
    gather(mb, kc, c0, kb0, a0);
    load_codes(mb + STEP, c1, e1);
    __syncthreads();
    for (; mb < m_end; mb += STEP) {   // mb is wave-uniform; rows past m_end carry code 0
      int c2[R], kb1[R];
      Extra e2[R];
      float a1[R][G];
      gather(mb + STEP, kc, c1, kb1, a1);
      load_codes(mb + 2 * STEP, c2, e2);
      finish(mb, kc, rows, c0, e0, kb0, a0);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        c0[r] = c1[r]; c1[r] = c2[r];
        e0[r] = e1[r]; e1[r] = e2[r];
        kb0[r] = kb1[r];
#pragma unroll
        for (int j = 0; j < G; ++j) a0[r][j] = a1[r][j];
      }
    }
  }
}

// Rows per workgroup (all of them unless that leaves the compute units short) and
// the grid of a resolve launch.
inline int resolve_grid(int B, int M, int N, int cols, int rows_step, int& panels, int& row_chunks,
                        int& rows_per, unsigned& grid) {
  panels = ceil_div(N, cols);
  row_chunks = 1;
  const int step = kResWaves * rows_step * (64 / cols);
  while ((int64_t)B * panels * row_chunks < 1024 && ceil_div(M, row_chunks) > 2 * step) row_chunks *= 2;
  rows_per = ceil_div(M, row_chunks);
  row_chunks = ceil_div(M, rows_per);
  const int64_t total = (int64_t)B * panels * row_chunks;
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  grid = (unsigned)total;
  return GENBMM_OK;
}

// max / prod-max: the maximum of the group's terms is the maximum of the cell (the
// group raised it last); descending k keeps the first term equal to it.
template <bool PROD>
struct MaxResolve {
  struct Extra {};
  elem_t* out;
  int32_t* idx;
  float* fa;  // optional: the two factors of the winning term per cell (product semiring)
  float* fb;
  __device__ __forceinline__ Extra load(long) const { return Extra{}; }
  __device__ __forceinline__ void none(long e) const {
    out[e] = to_elem<elem_t>(kFloor);
    if (fa) {
      fa[e] = 0.f;
      fb[e] = 0.f;
    }
  }
  __device__ __forceinline__ void cell(long e, int kb, const float (&av)[kResGroup], const float* br,
                                       int stride, int valid, int staged, Extra) const {
    constexpr int G = kResGroup;
    float t[G], bv[G];
#pragma unroll
    for (int j = 0; j < G; ++j) {
      bv[j] = br[min(j, staged - 1) * stride];
      t[j] = PROD ? av[j] * bv[j] : av[j] + bv[j];
      if (j >= valid) t[j] = -INFINITY;
    }
    float v = __builtin_fmaxf(__builtin_fmaxf(t[0], t[1]), t[2]);
    v = __builtin_fmaxf(__builtin_fmaxf(v, t[3]), t[4]);
    v = __builtin_fmaxf(__builtin_fmaxf(v, t[5]), t[6]);
    v = __builtin_fmaxf(v, t[7]);
    int first = G - 1;
#pragma unroll
    for (int j = G - 2; j >= 0; --j)
      if (t[j] == v) first = j;
    if (v == 0.f) {  // +0 and -0 compare equal: the value is the first one's
#pragma unroll
      for (int j = G - 1; j >= 0; --j)
        if (j == first) v = t[j];
    }
    idx[e] = kb + first;
    out[e] = to_elem<elem_t>(v);
    if (fa) {
      float sa = av[0], sb = bv[0];
#pragma unroll
      for (int j = 1; j < G; ++j) {
        sa = j == first ? av[j] : sa;
        sb = j == first ? bv[j] : sb;
      }
      fa[e] = sa;
      fb[e] = sb;
    }
  }
};

// TAIL: K is not a multiple of the group, the last group is cut at K.
template <bool PROD, int COLS, bool TAIL>
__global__ __launch_bounds__(kResWaves * 64, 4) void k_max_resolve(
    const elem_t* __restrict__ a, const elem_t* __restrict__ b, elem_t* __restrict__ out,
    int32_t* __restrict__ idx, float* __restrict__ fac_a, float* __restrict__ fac_b, int M, int K,
    int N, int panels, int row_chunks, int rows_per) {
  __shared__ float Bs[kResFloats];
  MaxResolve<PROD> op{out, idx, fac_a, fac_b};
  resolve_walk<COLS, TAIL, kResGroup, kResRows>(a, b, idx, op, M, K, N, panels, row_chunks, rows_per, Bs);
}

// ------------------------------------------------------------ sample forward
template <class C>
__global__ __launch_bounds__(C::NT) void k_sample_fwd(const DenseArgs p) {
  __shared__ __attribute__((aligned(16))) float As[C::KT * C::LDA];
  __shared__ __attribute__((aligned(16))) float Bs[C::KT * C::LDB];
  int batch, m0, n0;
  decode_tile<C>(p, batch, m0, n0);
  log_fwd_tile<C, true>(p, batch, m0, n0, As, Bs);
}

// Sampling sweep on top of a finished log-sum-exp (out) and the row / column
// maxima alpha, beta (stats): with EA = exp(a - alpha), EB = exp(b - beta) staged
// per tile, the unnormalised mass of term k is EA*EB and the target is
// u * S, S = exp(out - alpha - beta): one multiply per (m,k,n) instead of an
// exponential.  A tile in which any cell has S < 2^-40 (or is not finite) runs
// the online routine + exact sweep instead.
//
// TWO (shapes whose logbmm forward left EA, EB and a B*M*N scratch array in the
// workspace): two levels like the max forward.  The sweep reads EA / EB as they are,
// spends one multiply-add per term on the running rem = t - prefix sum, and looks at it
// only at the end of every group of kSampleGroup terms: its sign goes into the bit
// string (-> the group in which the prefix sum passes t), its smallest non-negative
// value (-> rem at the start of that group; non-negative floats order as unsigned
// integers and every negative one is larger) into the scratch array.
// k_sample_resolve then redoes the same multiply-adds for that one group.
constexpr int kSampleGroup = 8;

template <class C, bool TWO>
__global__ __launch_bounds__(C::NT, 2) void k_sample_sweep(const DenseArgs p,
                                                           const float* __restrict__ stats,
                                                           const float* __restrict__ ws_ea,
                                                           const float* __restrict__ ws_eb,
                                                           float* __restrict__ ws_rem) {
  __shared__ __attribute__((aligned(16))) float smem[C::KT * (C::LDA + C::LDB) + C::BM + C::BN];
  float* As = smem;
  float* Bs = As + C::KT * C::LDA;
  float* al = Bs + C::KT * C::LDB;
  float* be = al + C::BM;
  const int tid = threadIdx.x, tx = tid % C::TX, ty = tid / C::TX;
  int batch, m0, n0;
  decode_tile<C>(p, batch, m0, n0);
  const int M = p.M, K = p.K, N = p.N;
  using SrcT = std::conditional_t<TWO, float, elem_t>;  // the factors are fp32, the operands the caller's
  const SrcT *ab, *bb;
  if constexpr (TWO) {
    ab = ws_ea + (long)batch * M * K;
    bb = ws_eb + (long)batch * K * N;
  } else {
    ab = p.a + (long)batch * M * K;
    bb = p.b + (long)batch * K * N;
  }
  const elem_t* ob = p.out + (long)batch * M * N;
  const float* st = stats + (long)batch * (M + N);
  for (int t = tid; t < C::BM; t += C::NT) al[t] = (m0 + t < M) ? st[m0 + t] : 0.f;
  for (int t = tid; t < C::BN; t += C::NT) be[t] = (n0 + t < N) ? st[M + n0 + t] : 0.f;
  __syncthreads();

  // With the target t = u*S, the sampled index is the number of prefix sums that do
  // not exceed t (prefix sums never decrease).  Per cell: rem = t - prefix sum,
  // updated by one multiply-add per term; its sign bit (set once the prefix sum
  // has passed t; t - t = +0 keeps it clear) is shifted into a bit string by one
  // v_alignbit_b32 and the bits of a slab are counted once per slab.
  float rem[C::TM][C::TN];
  uint32_t bits[C::TM][C::TN];
  int ind[C::TM][C::TN];  // number of terms (TWO: groups) whose prefix sum exceeded t
  uint32_t low[TWO ? C::TM : 1][TWO ? C::TN : 1];  // TWO: smallest rem >= 0 seen at a group end
  const float lim = 40.f * kLn2 + 1e-3f;
  int bad = 0;
  const bool blocks = (N & 3) == 0;  // a lane's four adjacent cells then share one Philox block
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int jq = 0; jq < C::TN; jq += 4) {
      const int r = ty * C::TM + i, c0 = col_of<C>(tx, jq);
      const int m = m0 + r;
      float u[4] = {0.f, 0.f, 0.f, 0.f};
      if (m < M && n0 + c0 < N)
        philox_uniform4(((uint64_t)batch * M + m) * (uint64_t)N + (n0 + c0), blocks, p.seed, p.offset, u);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int j = jq + q, c = c0 + q, n = n0 + c;
        ind[i][j] = 0;
        rem[i][j] = 0.f;
        if (m < M && n < N) {
          const float e = al[r] + be[c] - ob[(long)m * N + n];   // -log S
          if (!(e <= lim) || !(e > -INFINITY)) bad = 1;
          // S = exp(-e) carries the rounding of `out` (2^-24 |out|) and the sweep adds the terms up in
          // another order than the forward did: a target that close to the total could lie beyond
          // the last prefix sum and never be passed, so every target is shrunk by 2^-17 of itself
          // (the boundaries between the terms move by 7.6e-6 of the total mass).
          rem[i][j] = (u[q] * (1.f - 0x1p-17f)) * fast_exp2(-e * kLog2e);
        }
        if (TWO) {
          low[i][j] = __float_as_uint(rem[i][j]);
          bits[i][j] = 0u;
        }
      }
    }
  if (__syncthreads_or(bad)) {  // workgroup-uniform
    log_fwd_tile<C, true>(p, batch, m0, n0, As, Bs);
    return;
  }

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
    for (int l = 0; l < (TWO ? 0 : TA::PER); ++l) {
      const float s = al[((tid + l * C::NT) / TA::C4) % C::BM];
      ta.r[l].x = fast_exp2((ta.r[l].x - s) * kLog2e); ta.r[l].y = fast_exp2((ta.r[l].y - s) * kLog2e);
      ta.r[l].z = fast_exp2((ta.r[l].z - s) * kLog2e); ta.r[l].w = fast_exp2((ta.r[l].w - s) * kLog2e);
    }
#pragma unroll
    for (int l = 0; l < (TWO ? 0 : TB::PER); ++l) {
      const float4 s = *reinterpret_cast<const float4*>(be + ((tid + l * C::NT) % TB::C4) * 4);
      tb.r[l].x = fast_exp2((tb.r[l].x - s.x) * kLog2e); tb.r[l].y = fast_exp2((tb.r[l].y - s.y) * kLog2e);
      tb.r[l].z = fast_exp2((tb.r[l].z - s.z) * kLog2e); tb.r[l].w = fast_exp2((tb.r[l].w - s.w) * kLog2e);
    }
    ta.sstore(As, tid);
    tb.sstore(Bs, tid);
    __syncthreads();
    if (k0 + C::KT < K) {
      ta.gload(ab, K, m0, k0 + C::KT, M, K, p.vec_a, tid);
      tb.gload(bb, N, n0, k0 + C::KT, N, K, p.vec_b, tid);
    }
    const int kn = min(C::KT, K - k0);
    static_assert(C::KT <= 32, "one bit per term of a slab");
    if (TWO) {
      // terms past K are zero (the loaders fill with 0): every slab is walked in full
      static_assert(C::KT % kSampleGroup == 0, "whole groups per slab");
#pragma unroll
      for (int g = 0; g < C::KT / kSampleGroup; ++g) {
#pragma unroll
        for (int kk = g * kSampleGroup; kk < (g + 1) * kSampleGroup; ++kk) {
          float av[C::TM], bv[C::TN];
          lds_frag<C::TM / 4>(As + kk * C::LDA, ty * C::TM, 4, av);
          lds_frag<C::TN / 4>(Bs + kk * C::LDB, tx * 4, C::TX * 4, bv);
#pragma unroll
          for (int i = 0; i < C::TM; ++i)
#pragma unroll
            for (int j = 0; j < C::TN; ++j) rem[i][j] = __builtin_fmaf(-av[i], bv[j], rem[i][j]);
        }
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
          for (int j = 0; j < C::TN; ++j) {
            const uint32_t rb = __float_as_uint(rem[i][j]);
            bits[i][j] = __builtin_amdgcn_alignbit(bits[i][j], rb, 31);
            low[i][j] = min(low[i][j], rb);
          }
      }
      // the bit string holds 32 groups
      constexpr int kFold = 32 / (C::KT / kSampleGroup);
      if ((k0 / C::KT) % kFold == kFold - 1 || k0 + C::KT >= K) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
          for (int j = 0; j < C::TN; ++j) {
            ind[i][j] += __builtin_popcount(bits[i][j]);
            bits[i][j] = 0u;
          }
      }
      continue;
    }
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
      for (int j = 0; j < C::TN; ++j) bits[i][j] = 0u;
    auto scan = [&](int kk) __attribute__((always_inline)) {
      float av[C::TM], bv[C::TN];
      lds_frag<C::TM / 4>(As + kk * C::LDA, ty * C::TM, 4, av);
      lds_frag<C::TN / 4>(Bs + kk * C::LDB, tx * 4, C::TX * 4, bv);
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
          rem[i][j] = __builtin_fmaf(-av[i], bv[j], rem[i][j]);
          bits[i][j] = __builtin_amdgcn_alignbit(bits[i][j], __float_as_uint(rem[i][j]), 31);
        }
    };
    if (kn == C::KT) {
#pragma unroll 4
      for (int kk = 0; kk < C::KT; ++kk) scan(kk);
    } else {
      for (int kk = 0; kk < kn; ++kk) scan(kk);
    }
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
      for (int j = 0; j < C::TN; ++j) ind[i][j] += __builtin_popcount(bits[i][j]);
  }
  if (TWO) {
    // group = groups walked - groups past t (none past t: rounding left the last prefix
    // sum a hair under t -> index 0, as below); the code -2 - group goes to idx, rem at
    // the start of that group to the scratch array
    const int walked = ((K + C::KT - 1) / C::KT) * (C::KT / kSampleGroup);
    float remv[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
      for (int j = 0; j < C::TN; ++j) {
        ind[i][j] = ind[i][j] == 0 ? 0 : -2 - (walked - ind[i][j]);
        remv[i][j] = __uint_as_float(low[i][j]);
      }
    store_tile_i<C>(p.idx + (long)batch * M * N, ind, m0, n0, M, N, p.vec_o, tx, ty);
    store_tile_f<C>(ws_rem + (long)batch * M * N, remv, m0, n0, M, N, p.vec_o && (reinterpret_cast<uintptr_t>(ws_rem) & 15u) == 0, tx, ty);
    return;
  }
  // index = K - (terms past t).  Rounding can leave the last prefix sum a hair under
  // u*S: no crossing -> index 0, as when the reference's walk never exceeds its draw
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j) ind[i][j] = ind[i][j] == 0 ? 0 : K - ind[i][j];
  store_tile_i<C>(p.idx + (long)batch * M * N, ind, m0, n0, M, N, p.vec_o, tx, ty);
}

// Second level of the sampling sweep: rem at the start of the group (G terms) goes
// through multiply-adds term by term; the index is the group's first term plus the
// number of terms after which rem is still >= 0 (rem only falls).
template <int G>
struct SampleResolve {
  typedef float Extra;
  const float* rem;
  int32_t* idx;
  int K;
  __device__ __forceinline__ float load(long e) const { return rem[e]; }
  __device__ __forceinline__ void none(long) const {}
  __device__ __forceinline__ void cell(long e, int kb, const float (&av)[G], const float* br, int stride,
                                       int valid, int staged, float r) const {
    uint32_t past = 0u;
#pragma unroll
    for (int j = 0; j < G; ++j) {
      const float ea = j < valid ? av[j] : 0.f;
      r = __builtin_fmaf(-ea, br[min(j, staged - 1) * stride], r);
      past = __builtin_amdgcn_alignbit(past, __float_as_uint(r), 31);
    }
    idx[e] = min(kb + G - __builtin_popcount(past), K - 1);
  }
};

template <int COLS, bool TAIL, int G>
__global__ __launch_bounds__(kResWaves * 64, 4) void k_sample_resolve(
    const float* __restrict__ ea, const float* __restrict__ eb, const float* __restrict__ remw,
    int32_t* __restrict__ idx, int* __restrict__ valid, int M, int K, int N, int panels,
    int row_chunks, int rows_per) {
  __shared__ float Bs[kResFloats];
  if (blockIdx.x == 0 && threadIdx.x == 0) *valid = 0;  // the 1/S array of the workspace is gone
  SampleResolve<G> op{remw, idx, K};
  // 16-term groups: two rows per step keep the pipelined values within the registers
  resolve_walk<COLS, TAIL, G, (G > 8 ? 2 : kResRows)>(ea, eb, idx, op, M, K, N, panels, row_chunks,
                                                     rows_per, Bs);
}

// ---------------------------------------------------------------- dispatch
template <class C, bool PROD>
int launch_max(DenseArgs p, float* factors, int B, int M, int K, int N, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<C>(p, B, M, K, N, grid)) return e;
  hipLaunchKernelGGL((k_max_fwd<C, PROD>), grid, dim3(C::NT), 0, s, p);
  if (int e = launch_status()) return e;
  if (K == 0) return GENBMM_OK;  // every code is -1 already
  float* fa = factors;
  float* fb = factors ? factors + (int64_t)B * M * N : nullptr;
  const int cols = K > 256 ? 32 : 64;  // 512 or 256 staged rows: one pass up to K = 512
  int panels, row_chunks, rows_per;
  unsigned rgrid;
  if (int e = resolve_grid(B, M, N, cols, kResRows, panels, row_chunks, rows_per, rgrid)) return e;
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(rgrid), dim3(kResWaves * 64), 0, s, p.a, p.b, p.out, p.idx, fa, fb,
                       M, K, N, panels, row_chunks, rows_per);
  };
  const bool tail = K % kMaxGroup != 0;
  if (cols == 64) {
    if (tail) go(k_max_resolve<PROD, 64, true>);
    else go(k_max_resolve<PROD, 64, false>);
  } else {
    if (tail) go(k_max_resolve<PROD, 32, true>);
    else go(k_max_resolve<PROD, 32, false>);
  }
  return launch_status();
}

#if GENBMM_ELEM == 0
// ------------------------------------------- max / prod-max: a long reduction in pieces
// Few result tiles and a long K would run on a few compute units, every tile being one
// workgroup's that walks all of K.  Such a problem is cut into pieces of K, a workgroup per
// 64 x 64 tile and piece, in two passes over a and b that need nothing beside out and idx:
//   pass 0  the maximum of a piece's terms joins out by an integer atomic on the value's bit pattern
//           (max of the pattern for values >= 0, min for negative ones: the order of floats);
//   pass 1  the lowest k of a piece whose term equals that maximum joins idx by an atomic minimum;
// then every cell forms the term of its index again (the value of the first term that attains
// the maximum, as the reference's walk keeps it - +0 and -0 compare equal, so the atomics
// cannot tell them apart) and, for the product semiring, stores its two factors.  Maximum and
// minimum commute: the result does not depend on the order in which the pieces arrive, and it is the
// sequential walk's (matmul_cuda_kernel.cu:47-75, :124-152) bit for bit.  A NaN term never wins
// (it is no maximum and equals nothing); k beyond a piece are staged as NaN.
constexpr int kCutTile = 64, kCutSlab = 16, kCutLda = 68;

// pieces of K for (B, M, K, N): 1 = no cut.  About two rounds of workgroups over the chip, pieces of
// at least 256 terms and a multiple of the slab.
inline int max_cut_pieces(int B, int M, int K, int N, int& per) {
  const int64_t tiles = (int64_t)B * ceil_div(M, kCutTile) * ceil_div(N, kCutTile);
  per = K;
  if (tiles <= 0 || tiles >= 128 || K < 2048) return 1;
  const int want = (int)std::min<int64_t>((511 + tiles) / tiles, K / 256);
  if (want < 2) return 1;
  per = ceil_div(ceil_div(K, want), kCutSlab) * kCutSlab;
  return ceil_div(K, per);
}

__global__ __launch_bounds__(256) void k_max_cut_init(float* __restrict__ out, int32_t* __restrict__ idx, long cells) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e < cells) {
    out[e] = kFloor;
    idx[e] = -1;
  }
}

// PASS 0 / 1 as above; one workgroup per tile and piece, a lane keeps 4 x 4 cells.
template <bool PROD, int PASS>
__global__ __launch_bounds__(256) void k_max_cut(const float* __restrict__ a, const float* __restrict__ b,
                                                float* __restrict__ out, int32_t* __restrict__ idx, int M, int K,
                                                int N, int tiles_m, int tiles_n, int pieces, int per) {
  __shared__ __attribute__((aligned(16))) float As[kCutSlab * kCutLda];   // [k][m]
  __shared__ __attribute__((aligned(16))) float Bs[kCutSlab * kCutTile];  // [k][n]
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int wg = xcd_renumber(blockIdx.x, gridDim.x);
  const int piece = wg % pieces, tile = wg / pieces;  // the pieces of a tile side by side: they share its cells
  const int per_item = tiles_m * tiles_n, batch = tile / per_item, rem = tile - batch * per_item;
  const int m0 = (rem / tiles_n) * kCutTile, n0 = (rem % tiles_n) * kCutTile;
  const int k_lo = piece * per, k_hi = min(K, k_lo + per);
  const float* ab = a + (long)batch * M * K;
  const float* bb = b + (long)batch * K * N;
  float* ob = out + (long)batch * M * N;
  int32_t* ib = idx + (long)batch * M * N;
  const int nslabs = (k_hi - k_lo + kCutSlab - 1) / kCutSlab;
  if (nslabs <= 0) return;

  const int ak = tid & 15, ar = tid >> 4, bn = tid & 63, bk = tid >> 6;
  float ra[4], rb[4];
  auto gload = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + ar + 16 * i, k = k0 + ak;
      ra[i] = k < k_hi ? (m < M ? ab[(long)m * K + k] : 0.f) : __builtin_nanf("");
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + bk + 4 * i, n = n0 + bn;
      rb[i] = (k < k_hi && n < N) ? bb[(long)k * N + n] : 0.f;
    }
  };
  auto sstore = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) As[ak * kCutLda + ar + 16 * i] = ra[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) Bs[(bk + 4 * i) * kCutTile + bn] = rb[i];
  };
  // the cells' state: the running maximum (pass 0) or the maximum to look for and the lowest k found
  float val[4][4];
  int cand[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      val[i][j] = PASS == 0 ? kFloor : ((m < M && n < N) ? ob[(long)m * N + n] : kFloor);
      cand[i][j] = 0x7fffffff;
    }
  // pass 1 walks its piece from the end, so that of the terms that match the lowest k is the one that stays
  auto slab_k0 = [&](int s) { return k_lo + (PASS == 0 ? s : nslabs - 1 - s) * kCutSlab; };
  gload(slab_k0(0));
  for (int s = 0; s < nslabs; ++s) {
    __syncthreads();
    sstore();
    __syncthreads();
    if (s + 1 < nslabs) gload(slab_k0(s + 1));
    const int k0 = slab_k0(s);
#pragma unroll
    for (int q = 0; q < kCutSlab; ++q) {
      const int kk = PASS == 0 ? q : kCutSlab - 1 - q;
      const float4 av = *reinterpret_cast<const float4*>(As + kk * kCutLda + ty * 4);
      const float4 bv = *reinterpret_cast<const float4*>(Bs + kk * kCutTile + tx * 4);
      const float a4[4] = {av.x, av.y, av.z, av.w}, b4[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float t = PROD ? __fmul_rn(a4[i], b4[j]) : __fadd_rn(a4[i], b4[j]);
          if (PASS == 0) val[i][j] = __builtin_fmaxf(val[i][j], t);
          else cand[i][j] = t == val[i][j] ? k0 + kk : cand[i][j];
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m >= M || n >= N) continue;
      const long e = (long)m * N + n;
      if (PASS == 0) {
        const float v = val[i][j] + 0.f;  // -0 joins as +0 (the value itself is formed again at the end)
        if (v > kFloor) {
          if (v >= 0.f) atomicMax(reinterpret_cast<int*>(ob + e), __float_as_int(v));
          else atomicMin(reinterpret_cast<unsigned*>(ob + e), __float_as_uint(v));
        }
      } else if (val[i][j] > kFloor && cand[i][j] != 0x7fffffff) {
        atomicMin(reinterpret_cast<unsigned*>(ib + e), (unsigned)cand[i][j]);  // -1, "none", is the largest
      }
    }
}

// the term of every cell's index again: the value, and the factors of the product semiring
template <bool PROD>
__global__ __launch_bounds__(256) void k_max_cut_finish(const float* __restrict__ a, const float* __restrict__ b,
                                                       float* __restrict__ out, const int32_t* __restrict__ idx,
                                                       float* __restrict__ fa, float* __restrict__ fb, int M, int K,
                                                       int N, long cells) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= cells) return;
  const int n = (int)(e % N);
  const long bm = e / N, batch = bm / M;
  const int k = idx[e];
  float av = 0.f, bv = 0.f;
  if (k >= 0) {
    av = a[bm * K + k];
    bv = b[(batch * K + k) * N + n];
    out[e] = PROD ? __fmul_rn(av, bv) : __fadd_rn(av, bv);
  }
  if (fa) {
    fa[e] = av;
    fb[e] = bv;
  }
}

template <bool PROD>
int launch_max_cut(const float* a, const float* b, float* out, int32_t* idx, float* factors, int B, int M, int K,
                   int N, int pieces, int per, hipStream_t s) {
  const long cells = (long)B * M * N;
  const int tiles_m = ceil_div(M, kCutTile), tiles_n = ceil_div(N, kCutTile);
  const unsigned grid = (unsigned)(B * tiles_m * tiles_n * pieces);  // below 128 tiles, at most 512 pieces
  const unsigned cgrid = (unsigned)((cells + 255) / 256);
  hipLaunchKernelGGL(k_max_cut_init, dim3(cgrid), dim3(256), 0, s, out, idx, cells);
  hipLaunchKernelGGL((k_max_cut<PROD, 0>), dim3(grid), dim3(256), 0, s, a, b, out, idx, M, K, N, tiles_m, tiles_n,
                     pieces, per);
  hipLaunchKernelGGL((k_max_cut<PROD, 1>), dim3(grid), dim3(256), 0, s, a, b, out, idx, M, K, N, tiles_m, tiles_n,
                     pieces, per);
  hipLaunchKernelGGL((k_max_cut_finish<PROD>), dim3(cgrid), dim3(256), 0, s, a, b, out, idx, factors,
                     factors ? factors + cells : nullptr, M, K, N, cells);
  return launch_status();
}
#endif

template <class C>
int launch_sample(DenseArgs p, int B, int M, int K, int N, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<C>(p, B, M, K, N, grid)) return e;
  hipLaunchKernelGGL((k_sample_fwd<C>), grid, dim3(C::NT), 0, s, p);
  return launch_status();
}

template <bool PROD>
int run_max(const elem_t* a, const elem_t* b, elem_t* out, int32_t* idx, float* factors, int B,
            int M, int K, int N, void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(idx, mn))
    return GENBMM_E_NULLPTR;
  if (mn == 0) return GENBMM_OK;
  DenseArgs p{};
  p.a = a; p.b = b; p.out = out; p.idx = idx;
  hipStream_t s = (hipStream_t)stream;
#if GENBMM_ELEM == 0
  {
    int per;
    const int pieces = max_cut_pieces(B, M, K, N, per);
    if (pieces > 1) return launch_max_cut<PROD>(a, b, out, idx, factors, B, M, K, N, pieces, per, s);
  }
#endif
  switch (pick_shape(B, M, N, false)) {
    case kBig: return launch_max<CfgBig, PROD>(p, factors, B, M, K, N, s);
    case kWide: return launch_max<CfgWide, PROD>(p, factors, B, M, K, N, s);
    case kMid: return launch_max<CfgMid, PROD>(p, factors, B, M, K, N, s);
    default: return launch_max<CfgSmall, PROD>(p, factors, B, M, K, N, s);
  }
}

template <class C>
int launch_sweep(DenseArgs p, const float* stats, int B, int M, int K, int N, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<C>(p, B, M, K, N, grid)) return e;
  hipLaunchKernelGGL((k_sample_sweep<C, false>), grid, dim3(C::NT), 0, s, p, stats,
                     (const float*)nullptr, (const float*)nullptr, (float*)nullptr);
  return launch_status();
}

// Second level of a sweep that left group codes (groups of `group` terms) in idx and
// rem in the workspace's scratch array.
template <int G>
int launch_sample_resolve(DenseArgs p, const LogFactors& f, int B, int M, int K, int N, hipStream_t s) {
  const int cols = K > 256 ? 32 : 64;
  int panels, row_chunks, rows_per;
  unsigned rgrid;
  if (int e = resolve_grid(B, M, N, cols, G > 8 ? 2 : kResRows, panels, row_chunks, rows_per, rgrid))
    return e;
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(rgrid), dim3(kResWaves * 64), 0, s, f.ea, f.eb, f.scratch, p.idx,
                       f.valid, M, K, N, panels, row_chunks, rows_per);
  };
  const bool tail = K % G != 0;
  if (cols == 64) {
    if (tail) go(k_sample_resolve<64, true, G>);
    else go(k_sample_resolve<64, false, G>);
  } else {
    if (tail) go(k_sample_resolve<32, true, G>);
    else go(k_sample_resolve<32, false, G>);
  }
  return launch_status();
}

// Two levels on the factors the logbmm forward left in the workspace, sweep on the
// vector ALU.
template <class C>
int launch_sweep_two(DenseArgs p, const float* stats, const LogFactors& f, int B, int M, int K,
                     int N, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<C>(p, B, M, K, N, grid)) return e;
  hipLaunchKernelGGL((k_sample_sweep<C, true>), grid, dim3(C::NT), 0, s, p, stats, f.ea, f.eb,
                     f.scratch);
  if (int e = launch_status()) return e;
  return launch_sample_resolve<kSampleGroup>(p, f, B, M, K, N, s);
}

int run_sample(const elem_t* a, const elem_t* b, elem_t* out, int32_t* idx, float* stats,
               uint64_t seed, uint64_t offset, int B, int M, int K, int N, void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(idx, mn))
    return GENBMM_E_NULLPTR;
  if (mn == 0) return GENBMM_OK;
  DenseArgs p{};
  p.a = a; p.b = b; p.out = out; p.idx = idx; p.seed = seed; p.offset = offset;
  hipStream_t s = (hipStream_t)stream;
  LogFactors f;
  // The vector-ALU sweeps take S = exp(out - alpha - beta) from `out` as stored; rounded to a
  // half type that is S within 2^-9 |out| at best, and targets u S past the true sum would be
  // common.  Half tensors therefore sweep only where 1/S itself is at hand in fp32 (the
  // matrix-core sweep) and walk exactly otherwise.
  // few result tiles and a long reduction: the forward cuts K into pieces, and so does the draw
  if (K > 0 && log_sample_cut_ok(stats, B, M, K, N))
    return log_sample_cut(a, b, out, idx, stats, seed, offset, B, M, K, N, s);
  const bool sweep = kElemF32 || (stats && log_fwd_writes_factors(stats, B, M, K, N, &f) && log_sample_mfma_ok(K));
  if (stats && K > 0 && sweep) {  // log-sum-exp by the logbmm forward, then the multiply-only sweep
    if (int e = log_fwd_with_factors(a, b, out, stats, B, M, K, N, s)) return e;
    if (log_fwd_writes_factors(stats, B, M, K, N, &f)) {
      if (log_sample_mfma_ok(K)) {  // sweep on the matrix cores, groups of 16 terms
        if (int e = log_sample_sweep_mfma(a, b, out, idx, stats, seed, offset, B, M, K, N, s)) return e;
        return launch_sample_resolve<16>(p, f, B, M, K, N, s);
      }
      switch (pick_shape(B, M, N, false)) {
        case kWide: return launch_sweep_two<CfgWide>(p, stats, f, B, M, K, N, s);
        default: return launch_sweep_two<CfgMid>(p, stats, f, B, M, K, N, s);
      }
    }
    switch (pick_shape(B, M, N, false)) {
      case kWide: return launch_sweep<CfgWide>(p, stats, B, M, K, N, s);
      case kMid: return launch_sweep<CfgMid>(p, stats, B, M, K, N, s);
      default: return launch_sweep<CfgSmall>(p, stats, B, M, K, N, s);
    }
  }
  switch (pick_shape(B, M, N, false)) {
    case kWide: return launch_sample<CfgWide>(p, B, M, K, N, s);
    case kMid: return launch_sample<CfgMid>(p, B, M, K, N, s);
    default: return launch_sample<CfgSmall>(p, B, M, K, N, s);
  }
}

}  // namespace
}  // namespace GENBMM_NS

extern "C" {

#if GENBMM_ELEM == 0
int genbmm_maxbmm_fwd_pieces(int B, int M, int K, int N) {
  using namespace GENBMM_NS;
  if (check_dense_dims(B, M, K, N) || (int64_t)B * M * N == 0) return 1;
  int per;
  return max_cut_pieces(B, M, K, N, per);
}
#endif

// One set per element type: genbmm_samplebmm_fwd, genbmm_samplebmm_fwd_f16, ..._bf16, ...
int GENBMM_API(samplebmm_fwd)(const GENBMM_NS::abi_t* a, const GENBMM_NS::abi_t* b, GENBMM_NS::abi_t* out,
                              int32_t* idx, float* stats, uint64_t seed, uint64_t offset, int B, int M,
                              int K, int N, void* stream) {
  using namespace GENBMM_NS;
  return run_sample(el(a), el(b), el(out), idx, stats, seed, offset, B, M, K, N, stream);
}

int GENBMM_API(maxbmm_fwd)(const GENBMM_NS::abi_t* a, const GENBMM_NS::abi_t* b, GENBMM_NS::abi_t* out,
                           int32_t* idx, int B, int M, int K, int N, void* stream) {
  using namespace GENBMM_NS;
  return run_max<false>(el(a), el(b), el(out), idx, nullptr, B, M, K, N, stream);
}

int GENBMM_API(prodmaxbmm_fwd)(const GENBMM_NS::abi_t* a, const GENBMM_NS::abi_t* b,
                               GENBMM_NS::abi_t* out, int32_t* idx, float* factors, int B, int M, int K,
                               int N, void* stream) {
  using namespace GENBMM_NS;
  return run_max<true>(el(a), el(b), el(out), idx, factors, B, M, K, N, stream);
}

}  // extern "C"
