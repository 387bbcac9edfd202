// Tile configuration, argument block and store helpers shared by the dense
// forward kernels, plus the online log-sum-exp tile routine (used by logbmm,
// by samplebmm and as the exact fallback of the factored logbmm path).
#pragma once

#include "common.h"

namespace GENBMM_NS {

template <int BM_, int BN_, int TM_, int TN_, int KT_>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, TM = TM_, TN = TN_, KT = KT_;
  static constexpr int TX = BN / TN, TY = BM / TM, NT = TX * TY;
  static constexpr int LDA = BM + kPad, LDB = BN + kPad;
  static_assert(TM % 4 == 0 && TN % 4 == 0 && KT % 4 == 0, "float4 fragments");
};

struct DenseArgs {
  const elem_t* a;
  const elem_t* b;
  elem_t* out;
  int32_t* idx;
  int M, K, N;
  int tiles_m, tiles_n;
  int vec_a, vec_b, vec_o;
  uint64_t seed, offset;
};

// Decode the 1-D workgroup id into (batch, m-tile, n-tile).
template <class C>
__device__ __forceinline__ void decode_tile(const DenseArgs& p, int& batch, int& m0, int& n0) {
  const int per = p.tiles_m * p.tiles_n;
  const int wg = xcd_renumber(blockIdx.x, gridDim.x);  // an XCD works on a contiguous run of tiles
  batch = wg / per;
  const int r = wg - batch * per;
  const int mt = r / p.tiles_n;
  m0 = mt * C::BM;
  n0 = (r - mt * p.tiles_n) * C::BN;
}

// Column of this lane's j-th output inside the tile: groups of four adjacent
// columns per lane, groups TX*4 apart, so a float4 LDS read / global write of
// consecutive lanes covers consecutive addresses.
template <class C>
__device__ __forceinline__ int col_of(int tx, int j) {
  return (j >> 2) * (C::TX * 4) + tx * 4 + (j & 3);
}

template <class C, class E>
__device__ __forceinline__ void store_tile_f(E* __restrict__ outb, const float (&v)[C::TM][C::TN],
                                             int m0, int n0, int M, int N, bool vec, int tx,
                                             int ty) {
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
    const int m = m0 + ty * C::TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int q = 0; q < C::TN / 4; ++q) {
      const int n = n0 + col_of<C>(tx, 4 * q);
      E* dst = outb + (long)m * N + n;
      if (vec && n + 3 < N) {
        st4a(dst, make_float4(v[i][4 * q], v[i][4 * q + 1], v[i][4 * q + 2], v[i][4 * q + 3]));
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) dst[e] = to_elem<E>(v[i][4 * q + e]);
      }
    }
  }
}

template <class C>
__device__ __forceinline__ void store_tile_i(int32_t* __restrict__ outb, const int (&v)[C::TM][C::TN],
                                             int m0, int n0, int M, int N, bool vec, int tx,
                                             int ty) {
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
    const int m = m0 + ty * C::TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int q = 0; q < C::TN / 4; ++q) {
      const int n = n0 + col_of<C>(tx, 4 * q);
      int32_t* dst = outb + (long)m * N + n;
      if (vec && n + 3 < N) {
        *reinterpret_cast<int4*>(dst) =
            make_int4(v[i][4 * q], v[i][4 * q + 1], v[i][4 * q + 2], v[i][4 * q + 3]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) dst[e] = v[i][4 * q + e];
      }
    }
  }
}

// ------------------------------------------------------- log / sample forward
// Online log-sum-exp.  Per K slab: (A) raise the running maximum of each cell
// over the slab, (B) rescale the running sum once, (C) add
// exp2((a+b)*log2e - max*log2e) for the slab.  a+b is rounded exactly as in
// the reference (matmul_cuda_kernel.cu:33,38); the maximum starts at -1e9
// (:31).  SAMPLE adds a second sweep over K that walks the CDF of
// softmax_k(a+b) against one Philox uniform per cell (reference :109-118).
template <class C, bool SAMPLE>
__device__ __forceinline__ void log_fwd_tile(const DenseArgs& p, int batch, int m0, int n0,
                                             float* __restrict__ As, float* __restrict__ Bs) {
  const int tid = threadIdx.x, tx = tid % C::TX, ty = tid / C::TX;
  const int M = p.M, K = p.K, N = p.N;
  const elem_t* ab = p.a + (long)batch * M * K;
  const elem_t* bb = p.b + (long)batch * K * N;

  float mx[C::TM][C::TN], acc[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
      mx[i][j] = kFloor;
      acc[i][j] = 0.f;
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

    // (A) slab maximum on top of the running maximum
    float nm[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
      for (int j = 0; j < C::TN; ++j) nm[i][j] = mx[i][j];
    auto pass_a = [&](int kk) __attribute__((always_inline)) {
      float av[C::TM], bv[C::TN];
      lds_frag<C::TM / 4>(As + kk * C::LDA, ty * C::TM, 4, av);
      lds_frag<C::TN / 4>(Bs + kk * C::LDB, tx * 4, C::TX * 4, bv);
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j) nm[i][j] = fmaxf(nm[i][j], av[i] + bv[j]);
    };
    if (kn == C::KT) {
#pragma unroll 4
      for (int kk = 0; kk < C::KT; ++kk) pass_a(kk);
    } else {
      for (int kk = 0; kk < kn; ++kk) pass_a(kk);
    }
    // (B) rescale; nm becomes -max*log2e for pass (C)
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
      for (int j = 0; j < C::TN; ++j) {
        acc[i][j] *= fast_exp2((mx[i][j] - nm[i][j]) * kLog2e);
        mx[i][j] = nm[i][j];
        nm[i][j] = -nm[i][j] * kLog2e;
      }
    // (C) accumulate
    auto pass_c = [&](int kk) __attribute__((always_inline)) {
      float av[C::TM], bv[C::TN];
      lds_frag<C::TM / 4>(As + kk * C::LDA, ty * C::TM, 4, av);
      lds_frag<C::TN / 4>(Bs + kk * C::LDB, tx * 4, C::TX * 4, bv);
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
          acc[i][j] += fast_exp2(__builtin_fmaf(av[i] + bv[j], kLog2e, nm[i][j]));
    };
    if (kn == C::KT) {
#pragma unroll 4
      for (int kk = 0; kk < C::KT; ++kk) pass_c(kk);
    } else {
      for (int kk = 0; kk < kn; ++kk) pass_c(kk);
    }
  }

  // out = log(sum) + max  (reference :41)
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j) mx[i][j] = logf(acc[i][j]) + mx[i][j];
  store_tile_f<C>(p.out + (long)batch * M * N, mx, m0, n0, M, N, p.vec_o, tx, ty);

  if (!SAMPLE) return;

  // ---- second sweep: inverse CDF.  rem = uniform - (mass scanned so far);
  // cell takes index k at the first k with rem > 0 and p_k > rem, which is
  // the reference's `total < r && total + p > r` with total = r - rem.
  // The masses exp(a + b - out) add up to 1 only within the rounding of `out` (2^-24 |out| in the
  // exponent), so a uniform that close to 1 can lie beyond the last prefix sum: such a cell takes
  // the last term that has any mass (`last`), not the reference's default of 0, which may name
  // a masked term.
  float rem[C::TM][C::TN];
  int ind[C::TM][C::TN], last[C::TM][C::TN];
  const bool blocks = (N & 3) == 0;  // a lane's four adjacent cells then share one Philox block
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int jq = 0; jq < C::TN; jq += 4) {
      const int m = m0 + ty * C::TM + i;
      const int n = n0 + col_of<C>(tx, jq);
      float u[4];
      philox_uniform4(((uint64_t)batch * M + m) * (uint64_t)N + n, blocks, p.seed, p.offset, u);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        rem[i][jq + q] = u[q];
        ind[i][jq + q] = 0;
        last[i][jq + q] = 0;
        mx[i][jq + q] = -mx[i][jq + q] * kLog2e;  // -out*log2e
      }
    }
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
    auto scan = [&](int kk) __attribute__((always_inline)) {
      float av[C::TM], bv[C::TN];
      lds_frag<C::TM / 4>(As + kk * C::LDA, ty * C::TM, 4, av);
      lds_frag<C::TN / 4>(Bs + kk * C::LDB, tx * 4, C::TX * 4, bv);
      const int k = k0 + kk;
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
          const float pk = fast_exp2(__builtin_fmaf(av[i] + bv[j], kLog2e, mx[i][j]));
          const float r = rem[i][j];
          if (r > 0.f && pk > r) ind[i][j] = k;
          if (pk > 0.f) last[i][j] = k;
          rem[i][j] = r - pk;
        }
    };
    if (kn == C::KT) {
#pragma unroll 4
      for (int kk = 0; kk < C::KT; ++kk) scan(kk);
    } else {
      for (int kk = 0; kk < kn; ++kk) scan(kk);
    }
  }
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
      if (rem[i][j] > 0.f) ind[i][j] = last[i][j];  // the walk never passed its target
  store_tile_i<C>(p.idx + (long)batch * M * N, ind, m0, n0, M, N, p.vec_o, tx, ty);
}


// ---------------------------------------------------------------- dispatch
using CfgBig = Cfg<128, 128, 8, 8, 16>;   // 256 lanes, 8x8 states per lane
using CfgWide = Cfg<64, 128, 4, 8, 16>;   // 256 lanes, 4x8
using CfgMid = Cfg<64, 64, 4, 4, 16>;     // 256 lanes, 4x4
using CfgSmall = Cfg<32, 32, 4, 4, 32>;   // one wave, 4x4

enum Shape { kBig, kWide, kMid, kSmall };

// Largest tile that still gives the 256 compute units a few workgroups each.
inline Shape pick_shape(int B, int M, int N, bool allow_big) {
  auto wgs = [&](int bm, int bn) { return (int64_t)B * ceil_div(M, bm) * ceil_div(N, bn); };
  if (M <= 32 && N <= 32) return kSmall;
  if (allow_big && M >= 128 && N >= 128 && wgs(128, 128) >= 1024) return kBig;
  if (M >= 64 && N >= 128 && wgs(64, 128) >= 512) return kWide;
  if (M > 32 || N > 32) return kMid;
  return kSmall;
}

template <class C>
inline int fill_args(DenseArgs& p, int B, int M, int K, int N, dim3& grid) {
  p.M = M; p.K = K; p.N = N;
  p.tiles_m = ceil_div(M, C::BM);
  p.tiles_n = ceil_div(N, C::BN);
  const int64_t total = (int64_t)B * p.tiles_m * p.tiles_n;
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  grid = dim3((unsigned)total, 1, 1);
  p.vec_a = (K % 4 == 0) && aligned16(p.a);
  p.vec_b = (N % 4 == 0) && aligned16(p.b);
  p.vec_o = (N % 4 == 0) && aligned16(p.out) && (p.idx == nullptr || aligned16(p.idx));
  return GENBMM_OK;
}

}  // namespace GENBMM_NS
