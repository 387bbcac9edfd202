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

namespace genbmm {
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
  const float* ab = p.a + (long)batch * M * K;
  const float* bb = p.b + (long)batch * K * N;

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

// Second level: group code -> value and index.  A workgroup owns kResCols columns
// of one batch item and a range of rows; the rows of b that the groups can point
// at are staged kResK at a time in LDS as [k][column], so that lane = column reads
// its own bank whatever k it needs, and the kMaxGroup values of a come from the
// row of a the whole wave shares.  The maximum of the group's terms is the
// maximum of the cell (the group raised it last); descending k keeps the first
// term equal to it.  Rows are taken kResRows at a time.
constexpr int kResCols = 64, kResK = 256, kResWaves = 8, kResRows = 4, kResStage = 8;
static_assert(kResK % kMaxGroup == 0, "a group lies in one staged chunk");
static_assert(kMaxGroup == 8, "the maximum chain below is written for eight terms");

typedef float float4_u __attribute__((ext_vector_type(4), aligned(4)));

// TAIL: K is not a multiple of the group, the last group is cut at K.
template <bool PROD, bool TAIL>
__global__ __launch_bounds__(kResWaves * 64) void k_max_resolve(
    const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ out,
    int32_t* __restrict__ idx, float* __restrict__ fac_a, float* __restrict__ fac_b, int M, int K,
    int N, int panels, int row_chunks, int rows_per) {
  __shared__ float Bs[kResK * kResCols];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int wg = blockIdx.x;
  const int panel = wg % panels;
  wg /= panels;
  const int chunk = wg % row_chunks;
  const int batch = wg / row_chunks;
  const int n = panel * kResCols + lane;
  const bool live = n < N;
  const int nc = min(n, N - 1);
  const int m_beg = chunk * rows_per, m_end = min(M, m_beg + rows_per);
  const float* ab = a + (long)batch * M * K;
  const float* bb = b + (long)batch * K * N;
  float* ob = out + (long)batch * M * N;
  int32_t* ib = idx + (long)batch * M * N;
  // optional: the two factors of the winning term per cell (product semiring)
  float* fa = fac_a ? fac_a + (long)batch * M * N : nullptr;
  float* fb = fac_b ? fac_b + (long)batch * M * N : nullptr;

  constexpr int R = kResRows, G = kMaxGroup, STEP = kResWaves * kResRows;
  // codes of R rows; 0 (nothing to do) outside the matrix
  auto load_codes = [&](int mb, int (&code)[R]) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int c = ib[(long)min(mb + r, M - 1) * N + nc];
      code[r] = (live && mb + r < m_end) ? c : 0;
    }
  };
  // first k of the group of each row (-1: not a group of the staged rows kc..) and
  // the group's values of a
  auto gather_a = [&](int mb, int kc, const int (&code)[R], int (&kb)[R], float (&av)[R][G])
                      __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int k = (-2 - code[r]) * G;
      const bool act = code[r] <= -2 && k >= kc && k < kc + kResK;
      kb[r] = act ? k : -1;
      const int ks = act ? k : kc;
      const float* ar = ab + (long)min(mb + r, M - 1) * K + ks;
      if (!TAIL) {
#pragma unroll
        for (int q = 0; q < G / 4; ++q) {
          const float4_u x = *reinterpret_cast<const float4_u*>(ar + 4 * q);
          av[r][4 * q] = x.x; av[r][4 * q + 1] = x.y; av[r][4 * q + 2] = x.z; av[r][4 * q + 3] = x.w;
        }
      } else {
#pragma unroll
        for (int j = 0; j < G; ++j) av[r][j] = ar[min(j, K - 1 - ks)];
      }
    }
  };
  auto finish = [&](int mb, int kc, int rows, const int (&code)[R], const int (&kb)[R],
                    const float (&av)[R][G]) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const long e = (long)(mb + r) * N + n;
      if (code[r] == -1 && kc == 0) {
        ob[e] = kFloor;
        if (fa) {
          fa[e] = 0.f;
          fb[e] = 0.f;
        }
      }
      if (kb[r] < 0) continue;
      const int rel = kb[r] - kc;
      const float* br = Bs + rel * kResCols + lane;
      float t[G], bv[G];
#pragma unroll
      for (int j = 0; j < G; ++j) {
        bv[j] = br[(TAIL ? min(j, rows - 1 - rel) : j) * kResCols];
        t[j] = PROD ? av[r][j] * bv[j] : av[r][j] + bv[j];
        if (TAIL && kb[r] + j >= K) t[j] = -INFINITY;
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
      ib[e] = kb[r] + first;
      ob[e] = v;
      if (fa) {
        float sa = av[r][0], sb = bv[0];
#pragma unroll
        for (int j = 1; j < G; ++j) {
          sa = j == first ? av[r][j] : sa;
          sb = j == first ? bv[j] : sb;
        }
        fa[e] = sa;
        fb[e] = sb;
      }
    }
  };

  for (int kc = 0; kc < K; kc += kResK) {
    const int rows = min(kResK, K - kc);
    int mb = m_beg + wave * R;
    int c0[R], c1[R], kb0[R];
    float a0[R][G];
    load_codes(mb, c0);
    __syncthreads();
    for (int r0 = wave; r0 < rows; r0 += kResWaves * kResStage) {
      float x[kResStage];
#pragma unroll
      for (int u = 0; u < kResStage; ++u)
        x[u] = bb[(long)(kc + min(r0 + u * kResWaves, rows - 1)) * N + nc];
#pragma unroll
      for (int u = 0; u < kResStage; ++u)
        if (r0 + u * kResWaves < rows) Bs[(r0 + u * kResWaves) * kResCols + lane] = x[u];
    }
    gather_a(mb, kc, c0, kb0, a0);
    load_codes(mb + STEP, c1);
    __syncthreads();
    // two sets of rows in flight: the codes two ahead and the values of a one ahead
    // are requested before the current rows are finished and stored
    for (; mb < m_end; mb += STEP) {
      int c2[R], kb1[R];
      float a1[R][G];
      gather_a(mb + STEP, kc, c1, kb1, a1);
      load_codes(mb + 2 * STEP, c2);
      finish(mb, kc, rows, c0, kb0, a0);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        c0[r] = c1[r];
        c1[r] = c2[r];
        kb0[r] = kb1[r];
#pragma unroll
        for (int j = 0; j < G; ++j) a0[r][j] = a1[r][j];
      }
    }
  }
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
template <class C>
__global__ __launch_bounds__(C::NT, 2) void k_sample_sweep(const DenseArgs p,
                                                           const float* __restrict__ stats) {
  __shared__ __attribute__((aligned(16))) float smem[C::KT * (C::LDA + C::LDB) + C::BM + C::BN];
  float* As = smem;
  float* Bs = As + C::KT * C::LDA;
  float* al = Bs + C::KT * C::LDB;
  float* be = al + C::BM;
  const int tid = threadIdx.x, tx = tid % C::TX, ty = tid / C::TX;
  int batch, m0, n0;
  decode_tile<C>(p, batch, m0, n0);
  const int M = p.M, K = p.K, N = p.N;
  const float* ab = p.a + (long)batch * M * K;
  const float* bb = p.b + (long)batch * K * N;
  const float* ob = p.out + (long)batch * M * N;
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
  int ind[C::TM][C::TN];  // number of terms whose prefix sum exceeded t
  const float lim = 40.f * kLn2 + 1e-3f;
  int bad = 0;
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
      const int r = ty * C::TM + i, c = col_of<C>(tx, j);
      const int m = m0 + r, n = n0 + c;
      ind[i][j] = 0;
      rem[i][j] = 0.f;
      if (m < M && n < N) {
        const float e = al[r] + be[c] - ob[(long)m * N + n];   // -log S
        if (!(e <= lim) || !(e > -INFINITY)) bad = 1;
        const uint64_t cell = ((uint64_t)batch * M + m) * (uint64_t)N + n;
        rem[i][j] = philox_uniform(cell, p.seed, p.offset) * fast_exp2(-e * kLog2e);
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
    for (int l = 0; l < TA::PER; ++l) {
      const float s = al[((tid + l * C::NT) / TA::C4) % C::BM];
      ta.r[l].x = fast_exp2((ta.r[l].x - s) * kLog2e); ta.r[l].y = fast_exp2((ta.r[l].y - s) * kLog2e);
      ta.r[l].z = fast_exp2((ta.r[l].z - s) * kLog2e); ta.r[l].w = fast_exp2((ta.r[l].w - s) * kLog2e);
    }
#pragma unroll
    for (int l = 0; l < TB::PER; ++l) {
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
  // index = K - (terms past t).  Rounding can leave the last prefix sum a hair under
  // u*S: no crossing -> index 0, as when the reference's walk never exceeds its draw
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j) ind[i][j] = ind[i][j] == 0 ? 0 : K - ind[i][j];
  store_tile_i<C>(p.idx + (long)batch * M * N, ind, m0, n0, M, N, p.vec_o, tx, ty);
}

// ---------------------------------------------------------------- dispatch
template <class C, bool PROD>
int launch_max(DenseArgs p, float* factors, int B, int M, int K, int N, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<C>(p, B, M, K, N, grid)) return e;
  hipLaunchKernelGGL((k_max_fwd<C, PROD>), grid, dim3(C::NT), 0, s, p);
  if (int e = launch_status()) return e;
  if (K == 0) return GENBMM_OK;  // every code is -1 already
  // rows per workgroup: all of them unless that leaves the compute units short
  const int panels = ceil_div(N, kResCols);
  int row_chunks = 1;
  while ((int64_t)B * panels * row_chunks < 1024 && ceil_div(M, row_chunks) > 2 * kResWaves * kResRows)
    row_chunks *= 2;
  const int rows_per = ceil_div(M, row_chunks);
  row_chunks = ceil_div(M, rows_per);
  const int64_t total = (int64_t)B * panels * row_chunks;
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  float* fa = factors;
  float* fb = factors ? factors + (int64_t)B * M * N : nullptr;
  if (K % kMaxGroup == 0)
    hipLaunchKernelGGL((k_max_resolve<PROD, false>), dim3((unsigned)total), dim3(kResWaves * 64), 0,
                       s, p.a, p.b, p.out, p.idx, fa, fb, M, K, N, panels, row_chunks, rows_per);
  else
    hipLaunchKernelGGL((k_max_resolve<PROD, true>), dim3((unsigned)total), dim3(kResWaves * 64), 0,
                       s, p.a, p.b, p.out, p.idx, fa, fb, M, K, N, panels, row_chunks, rows_per);
  return launch_status();
}

template <class C>
int launch_sample(DenseArgs p, int B, int M, int K, int N, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<C>(p, B, M, K, N, grid)) return e;
  hipLaunchKernelGGL((k_sample_fwd<C>), grid, dim3(C::NT), 0, s, p);
  return launch_status();
}

template <bool PROD>
int run_max(const float* a, const float* b, float* out, int32_t* idx, float* factors, int B,
            int M, int K, int N, void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(idx, mn))
    return GENBMM_E_NULLPTR;
  if (mn == 0) return GENBMM_OK;
  DenseArgs p{};
  p.a = a; p.b = b; p.out = out; p.idx = idx;
  hipStream_t s = (hipStream_t)stream;
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
  hipLaunchKernelGGL((k_sample_sweep<C>), grid, dim3(C::NT), 0, s, p, stats);
  return launch_status();
}

int run_sample(const float* a, const float* b, float* out, int32_t* idx, float* stats,
               uint64_t seed, uint64_t offset, int B, int M, int K, int N, void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(idx, mn))
    return GENBMM_E_NULLPTR;
  if (mn == 0) return GENBMM_OK;
  DenseArgs p{};
  p.a = a; p.b = b; p.out = out; p.idx = idx; p.seed = seed; p.offset = offset;
  hipStream_t s = (hipStream_t)stream;
  if (stats && K > 0) {  // log-sum-exp by the logbmm forward, then the multiply-only sweep
    if (int e = genbmm_logbmm_fwd(a, b, out, stats, B, M, K, N, stream)) return e;
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
}  // namespace genbmm

extern "C" {

int genbmm_samplebmm_fwd(const float* a, const float* b, float* out, int32_t* idx, float* stats,
                         uint64_t seed, uint64_t offset, int B, int M, int K, int N,
                         void* stream) {
  return genbmm::run_sample(a, b, out, idx, stats, seed, offset, B, M, K, N, stream);
}

int genbmm_maxbmm_fwd(const float* a, const float* b, float* out, int32_t* idx, int B, int M,
                      int K, int N, void* stream) {
  return genbmm::run_max<false>(a, b, out, idx, nullptr, B, M, K, N, stream);
}

int genbmm_prodmaxbmm_fwd(const float* a, const float* b, float* out, int32_t* idx,
                          float* factors, int B, int M, int K, int N, void* stream) {
  return genbmm::run_max<true>(a, b, out, idx, factors, B, M, K, N, stream);
}

}  // extern "C"
