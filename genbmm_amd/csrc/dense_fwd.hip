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
#include "common.h"

namespace genbmm {
namespace {

template <int BM_, int BN_, int TM_, int TN_, int KT_>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, TM = TM_, TN = TN_, KT = KT_;
  static constexpr int TX = BN / TN, TY = BM / TM, NT = TX * TY;
  static constexpr int LDA = BM + kPad, LDB = BN + kPad;
  static_assert(TM % 4 == 0 && TN % 4 == 0 && KT % 4 == 0, "float4 fragments");
};

struct DenseArgs {
  const float* a;
  const float* b;
  float* out;
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
  const int wg = blockIdx.x;
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

template <class C>
__device__ __forceinline__ void store_tile_f(float* __restrict__ outb, const float (&v)[C::TM][C::TN],
                                             int m0, int n0, int M, int N, bool vec, int tx,
                                             int ty) {
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
    const int m = m0 + ty * C::TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int q = 0; q < C::TN / 4; ++q) {
      const int n = n0 + col_of<C>(tx, 4 * q);
      float* dst = outb + (long)m * N + n;
      if (vec && n + 3 < N) {
        *reinterpret_cast<float4*>(dst) =
            make_float4(v[i][4 * q], v[i][4 * q + 1], v[i][4 * q + 2], v[i][4 * q + 3]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) dst[e] = v[i][4 * q + e];
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

// ------------------------------------------------------- max / prod-max forward
// Reference: max_cuda_forward_kernel (matmul_cuda_kernel.cu:47-75) and
// prod_max_cuda_forward_kernel (:124-152): ascending k, strict '>', running
// maximum starts at -1e9 with index -1.
template <class C, bool PROD>
__global__ __launch_bounds__(C::NT) void k_max_fwd(const DenseArgs p) {
  __shared__ __attribute__((aligned(16))) float As[C::KT * C::LDA];
  __shared__ __attribute__((aligned(16))) float Bs[C::KT * C::LDB];
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
    auto step = [&](int kk) __attribute__((always_inline)) {
      float av[C::TM], bv[C::TN];
      lds_frag<C::TM / 4>(As + kk * C::LDA, ty * C::TM, 4, av);
      lds_frag<C::TN / 4>(Bs + kk * C::LDB, tx * 4, C::TX * 4, bv);
      const int k = k0 + kk;
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
          const float t = PROD ? av[i] * bv[j] : av[i] + bv[j];
          if (t > mx[i][j]) {
            mx[i][j] = t;
            ind[i][j] = k;
          }
        }
    };
    if (kn == C::KT) {
#pragma unroll 4
      for (int kk = 0; kk < C::KT; ++kk) step(kk);
    } else {
      for (int kk = 0; kk < kn; ++kk) step(kk);
    }
  }
  store_tile_f<C>(p.out + (long)batch * M * N, mx, m0, n0, M, N, p.vec_o, tx, ty);
  store_tile_i<C>(p.idx + (long)batch * M * N, ind, m0, n0, M, N, p.vec_o, tx, ty);
}

// ------------------------------------------------------- log / sample forward
// Online log-sum-exp.  Per K slab: (A) raise the running maximum of each cell
// over the slab, (B) rescale the running sum once, (C) add
// exp2((a+b)*log2e - max*log2e) for the slab.  a+b is rounded exactly as in
// the reference (matmul_cuda_kernel.cu:33,38); the maximum starts at -1e9
// (:31).  SAMPLE adds a second sweep over K that walks the CDF of
// softmax_k(a+b) against one Philox uniform per cell (reference :109-118).
template <class C, bool SAMPLE>
__global__ __launch_bounds__(C::NT) void k_log_fwd(const DenseArgs p) {
  __shared__ __attribute__((aligned(16))) float As[C::KT * C::LDA];
  __shared__ __attribute__((aligned(16))) float Bs[C::KT * C::LDB];
  const int tid = threadIdx.x, tx = tid % C::TX, ty = tid / C::TX;
  int batch, m0, n0;
  decode_tile<C>(p, batch, m0, n0);
  const int M = p.M, K = p.K, N = p.N;
  const float* ab = p.a + (long)batch * M * K;
  const float* bb = p.b + (long)batch * K * N;

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
  float rem[C::TM][C::TN];
  int ind[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
      const int m = m0 + ty * C::TM + i;
      const int n = n0 + col_of<C>(tx, j);
      const uint64_t cell = ((uint64_t)batch * M + m) * (uint64_t)N + n;
      rem[i][j] = philox_uniform(cell, p.seed, p.offset);
      ind[i][j] = 0;
      mx[i][j] = -mx[i][j] * kLog2e;  // -out*log2e
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
int fill_args(DenseArgs& p, int B, int M, int K, int N, dim3& grid) {
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

template <class C, bool PROD>
int launch_max(DenseArgs p, int B, int M, int K, int N, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<C>(p, B, M, K, N, grid)) return e;
  hipLaunchKernelGGL((k_max_fwd<C, PROD>), grid, dim3(C::NT), 0, s, p);
  return launch_status();
}

template <class C, bool SAMPLE>
int launch_log(DenseArgs p, int B, int M, int K, int N, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<C>(p, B, M, K, N, grid)) return e;
  hipLaunchKernelGGL((k_log_fwd<C, SAMPLE>), grid, dim3(C::NT), 0, s, p);
  return launch_status();
}

template <bool PROD>
int run_max(const float* a, const float* b, float* out, int32_t* idx, int B, int M, int K, int N,
            void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(idx, mn))
    return GENBMM_E_NULLPTR;
  if (mn == 0) return GENBMM_OK;
  DenseArgs p{};
  p.a = a; p.b = b; p.out = out; p.idx = idx;
  hipStream_t s = (hipStream_t)stream;
  switch (pick_shape(B, M, N, true)) {
    case kBig: return launch_max<CfgBig, PROD>(p, B, M, K, N, s);
    case kWide: return launch_max<CfgWide, PROD>(p, B, M, K, N, s);
    case kMid: return launch_max<CfgMid, PROD>(p, B, M, K, N, s);
    default: return launch_max<CfgSmall, PROD>(p, B, M, K, N, s);
  }
}

template <bool SAMPLE>
int run_log(const float* a, const float* b, float* out, int32_t* idx, uint64_t seed,
            uint64_t offset, int B, int M, int K, int N, void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || (SAMPLE && missing(idx, mn)))
    return GENBMM_E_NULLPTR;
  if (mn == 0) return GENBMM_OK;
  DenseArgs p{};
  p.a = a; p.b = b; p.out = out; p.idx = idx; p.seed = seed; p.offset = offset;
  hipStream_t s = (hipStream_t)stream;
  switch (pick_shape(B, M, N, false)) {
    case kWide: return launch_log<CfgWide, SAMPLE>(p, B, M, K, N, s);
    case kMid: return launch_log<CfgMid, SAMPLE>(p, B, M, K, N, s);
    default: return launch_log<CfgSmall, SAMPLE>(p, B, M, K, N, s);
  }
}

}  // namespace
}  // namespace genbmm

extern "C" {

int genbmm_logbmm_fwd(const float* a, const float* b, float* out, int B, int M, int K, int N,
                      void* stream) {
  return genbmm::run_log<false>(a, b, out, nullptr, 0, 0, B, M, K, N, stream);
}

int genbmm_samplebmm_fwd(const float* a, const float* b, float* out, int32_t* idx, uint64_t seed,
                         uint64_t offset, int B, int M, int K, int N, void* stream) {
  return genbmm::run_log<true>(a, b, out, idx, seed, offset, B, M, K, N, stream);
}

int genbmm_maxbmm_fwd(const float* a, const float* b, float* out, int32_t* idx, int B, int M,
                      int K, int N, void* stream) {
  return genbmm::run_max<false>(a, b, out, idx, B, M, K, N, stream);
}

int genbmm_prodmaxbmm_fwd(const float* a, const float* b, float* out, int32_t* idx, int B, int M,
                          int K, int N, void* stream) {
  return genbmm::run_max<true>(a, b, out, idx, B, M, K, N, stream);
}

}  // extern "C"
