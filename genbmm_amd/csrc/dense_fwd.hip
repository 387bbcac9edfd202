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

// ------------------------------------------------------------ sample forward
template <class C>
__global__ __launch_bounds__(C::NT) void k_sample_fwd(const DenseArgs p) {
  __shared__ __attribute__((aligned(16))) float As[C::KT * C::LDA];
  __shared__ __attribute__((aligned(16))) float Bs[C::KT * C::LDB];
  int batch, m0, n0;
  decode_tile<C>(p, batch, m0, n0);
  log_fwd_tile<C, true>(p, batch, m0, n0, As, Bs);
}

// ---------------------------------------------------------------- dispatch
template <class C, bool PROD>
int launch_max(DenseArgs p, int B, int M, int K, int N, hipStream_t s) {
  dim3 grid;
  if (int e = fill_args<C>(p, B, M, K, N, grid)) return e;
  hipLaunchKernelGGL((k_max_fwd<C, PROD>), grid, dim3(C::NT), 0, s, p);
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
  switch (pick_shape(B, M, N, false)) {
    case kBig: return launch_max<CfgBig, PROD>(p, B, M, K, N, s);
    case kWide: return launch_max<CfgWide, PROD>(p, B, M, K, N, s);
    case kMid: return launch_max<CfgMid, PROD>(p, B, M, K, N, s);
    default: return launch_max<CfgSmall, PROD>(p, B, M, K, N, s);
  }
}

int run_sample(const float* a, const float* b, float* out, int32_t* idx, uint64_t seed,
               uint64_t offset, int B, int M, int K, int N, void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(a, mk) || missing(b, kn) || missing(out, mn) || missing(idx, mn))
    return GENBMM_E_NULLPTR;
  if (mn == 0) return GENBMM_OK;
  DenseArgs p{};
  p.a = a; p.b = b; p.out = out; p.idx = idx; p.seed = seed; p.offset = offset;
  hipStream_t s = (hipStream_t)stream;
  switch (pick_shape(B, M, N, false)) {
    case kWide: return launch_sample<CfgWide>(p, B, M, K, N, s);
    case kMid: return launch_sample<CfgMid>(p, B, M, K, N, s);
    default: return launch_sample<CfgSmall>(p, B, M, K, N, s);
  }
}

}  // namespace
}  // namespace genbmm

extern "C" {

int genbmm_samplebmm_fwd(const float* a, const float* b, float* out, int32_t* idx, uint64_t seed,
                         uint64_t offset, int B, int M, int K, int N, void* stream) {
  return genbmm::run_sample(a, b, out, idx, seed, offset, B, M, K, N, stream);
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
