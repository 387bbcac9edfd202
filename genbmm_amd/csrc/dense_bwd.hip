// Dense semiring batched matmul: the arg-max backward kernels (gfx950).
#include "common.h"

namespace GENBMM_NS {
namespace {

// ===================================================== argmax backward
//
// maxbmm / samplebmm:  grad_a[m,k] = sum_n [k == idx[m,n]] g[m,n]
//                      grad_b[k,n] = sum_m [k == idx[m,n]] g[m,n]
// prodmaxbmm: the terms are b[k,n]*g[m,n] and a[m,k]*g[m,n].
// (reference matmul_cuda_kernel.cu:336-456: one thread per gradient cell
// scanning the whole reduction axis, O(M*K*N).)  Here a lane owns a row m (resp.
// column n) and a range of k, walks the row once in ascending n (resp. the column
// in ascending m) and adds each term whose idx falls into its range to that
// cell of an LDS-resident accumulator; the additions hitting a given cell
// therefore happen in the reference's order, so the result is bit-identical, in
// O(M*N) work.  Products are rounded before the add (the build uses
// -ffp-contract=on: no fusion across statements).
constexpr int kKC = 128;  // cells of the reduction axis per lane

// The 64 lanes of a workgroup are (line, part): 64 >> ps lines (rows m of grad_a,
// columns n of grad_b) times 2^ps parts of kKC consecutive k, so that one workgroup
// covers every k of its lines (up to 64 * kKC; longer K: further workgroups) and idx
// and g are read from memory once - the lanes of a line read the same addresses.
// Each lane walks its whole line and adds the terms whose k falls into its part.

// grad_a: line = row m.  The row is read 16 cells at a time (int4 / float4 when the
// rows are 16-byte aligned), then the 16 additions are made in order.
constexpr int kArgAccA = 64 * kKC + 64 + 64, kArgAccB = kKC * 64 + 64;  // floats of LDS
// (blk: the workgroup's number among those of grad_a; accs: kArgAccA floats of LDS)
template <int PROD>
__device__ __forceinline__ void argmax_bwd_a_block(float* __restrict__ accs, int blk,
                                                   const elem_t* __restrict__ bmat,
                                                   const float* __restrict__ fac,
                                                   const int32_t* __restrict__ idx,
                                                   const elem_t* __restrict__ g,
                                                   elem_t* __restrict__ grad_a, int M, int K,
                                                   int N, int row_tiles, int k_chunks, int ps,
                                                   int vec) {
  const int lane = threadIdx.x, parts = 1 << ps, lines = 64 >> ps;
  const int part = lane & (parts - 1), line = lane >> ps;
  const int spare = 64 * kKC + 64 + lane;
  const int kc_id = blk % k_chunks, rt = blk / k_chunks;
  const int batch = rt / row_tiles;
  const int m0 = (rt - batch * row_tiles) * lines;
  const int kw = parts * kKC;                       // k covered by the workgroup
  const int w0 = kc_id * kw, c0 = w0 + part * kKC;  // first k of the workgroup / of this lane
  const int kc = min(kKC, K - c0);                  // <= 0: the part lies beyond K
  const int m = m0 + line;
  const bool live = m < M;
  const int32_t* irow = idx + ((long)batch * M + (live ? m : 0)) * N;
  const elem_t* grow = g + ((long)batch * M + (live ? m : 0)) * N;
  const elem_t* bb = PROD == 1 ? bmat + (long)batch * K * N : nullptr;
  const float* frow = PROD == 2 ? fac + ((long)batch * M + (live ? m : 0)) * N : nullptr;
  const int base = line * (kw + 1) + part * kKC;
  float* mine = accs + base;
  for (int kk = 0; kk < kKC; ++kk) mine[kk] = 0.f;
  accs[spare] = 0.f;
  auto slot = [&](int ki) __attribute__((always_inline)) {
    const int k = ki - c0;
    return (k >= 0 && k < kc) ? base + k : spare;
  };
  // the term of cell n: g, times b[idx, n] for the product semiring (read only when
  // the index falls into this lane's k range)
  auto term = [&](int n, int ki, float gv) __attribute__((always_inline)) {
    const int k = ki - c0;
    if (PROD == 1 && k >= 0 && k < kc) return __fmul_rn(bb[(long)ki * N + n], gv);
    return gv;
  };
  auto add = [&](int ki, float v) __attribute__((always_inline)) {
    const int k = ki - c0;
    if (k >= 0 && k < kc) mine[k] = __fadd_rn(mine[k], v);
  };
  if (live) {
    int n = 0;
    if (vec) {
      for (; n + 16 <= N; n += 16) {
        int4 iv[4];
        float4 gv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          iv[q] = *reinterpret_cast<const int4*>(irow + n + 4 * q);
          gv[q] = ld4a(grow + n + 4 * q);
        }
        if (PROD == 2) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float4 f = *reinterpret_cast<const float4*>(frow + n + 4 * q);
            gv[q].x = __fmul_rn(f.x, gv[q].x);
            gv[q].y = __fmul_rn(f.y, gv[q].y);
            gv[q].z = __fmul_rn(f.z, gv[q].z);
            gv[q].w = __fmul_rn(f.w, gv[q].w);
          }
        }
        // all sixteen factors are requested before the first (ordered) addition
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          gv[q].x = term(n + 4 * q, iv[q].x, gv[q].x);
          gv[q].y = term(n + 4 * q + 1, iv[q].y, gv[q].y);
          gv[q].z = term(n + 4 * q + 2, iv[q].z, gv[q].z);
          gv[q].w = term(n + 4 * q + 3, iv[q].w, gv[q].w);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int sl[4] = {slot(iv[q].x), slot(iv[q].y), slot(iv[q].z), slot(iv[q].w)};
          const float tv[4] = {gv[q].x, gv[q].y, gv[q].z, gv[q].w};
          add4_ordered(accs, sl, tv);
        }
      }
    }
    for (; n < N; ++n)
      add(irow[n], PROD == 2 ? __fmul_rn(frow[n], grow[n]) : term(n, irow[n], grow[n]));
  }
  __syncthreads();
  const int rows = min(lines, M - m0), kn = min(kw, K - w0);
  for (int r = 0; r < rows; ++r) {
    elem_t* dst = grad_a + ((long)batch * M + m0 + r) * K + w0;
    for (int kk = lane; kk < kn; kk += 64) dst[kk] = to_elem<elem_t>(accs[r * (kw + 1) + kk]);
  }
}

// grad_b: line = column n; the column is read 16 rows at a time, then added in order.
// Accumulators are [k][line].
// (blk: the workgroup's number among those of grad_b; accs: kArgAccB floats of LDS)
template <int PROD>
__device__ __forceinline__ void argmax_bwd_b_block(float* __restrict__ accs, int blk,
                                                   const elem_t* __restrict__ amat,
                                                   const float* __restrict__ fac,
                                                   const int32_t* __restrict__ idx,
                                                   const elem_t* __restrict__ g,
                                                   elem_t* __restrict__ grad_b, int M, int K,
                                                   int N, int col_tiles, int k_chunks, int ps) {
  const int lane = threadIdx.x, parts = 1 << ps, lines = 64 >> ps;
  const int part = lane & (parts - 1), line = lane >> ps;
  const int spare = kKC * 64 + lane;
  const int kc_id = blk % k_chunks, ct = blk / k_chunks;
  const int batch = ct / col_tiles;
  const int n0 = (ct - batch * col_tiles) * lines, n = n0 + line;
  const int kw = parts * kKC;
  const int w0 = kc_id * kw, c0 = w0 + part * kKC;
  const int kc = min(kKC, K - c0);
  const bool live = n < N;
  const int nn = live ? n : N - 1;
  const int32_t* icol = idx + (long)batch * M * N + nn;
  const elem_t* gcol = g + (long)batch * M * N + nn;
  const elem_t* ab = PROD == 1 ? amat + (long)batch * M * K : nullptr;
  const float* fcol = PROD == 2 ? fac + (long)batch * M * N + nn : nullptr;
  const int base = (part * kKC) * lines + line;  // cell k of this lane: accs[base + k * lines]
  float* mine = accs + base;
  for (int kk = 0; kk < kKC; ++kk) mine[kk * lines] = 0.f;
  accs[spare] = 0.f;
  auto slot = [&](int ki) __attribute__((always_inline)) {
    const int k = ki - c0;
    return (k >= 0 && k < kc) ? base + k * lines : spare;
  };
  auto term = [&](int m, int ki, float gv) __attribute__((always_inline)) {
    const int k = ki - c0;
    if (PROD == 1 && k >= 0 && k < kc) return __fmul_rn(ab[(long)m * K + ki], gv);
    if (PROD == 2) return __fmul_rn(fcol[(long)m * N], gv);
    return gv;
  };
  auto add = [&](int ki, float v) __attribute__((always_inline)) {
    const int k = ki - c0;
    if (k >= 0 && k < kc) mine[k * lines] = __fadd_rn(mine[k * lines], v);
  };
  if (live) {
    int m = 0;
    for (; m + 16 <= M; m += 16) {
      int iv[16];
      float gv[16];
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        iv[q] = icol[(long)(m + q) * N];
        gv[q] = gcol[(long)(m + q) * N];
      }
#pragma unroll
      for (int q = 0; q < 16; ++q) gv[q] = term(m + q, iv[q], gv[q]);
#pragma unroll
      for (int q = 0; q < 16; q += 4) {
        const int sl[4] = {slot(iv[q]), slot(iv[q + 1]), slot(iv[q + 2]), slot(iv[q + 3])};
        const float tv[4] = {gv[q], gv[q + 1], gv[q + 2], gv[q + 3]};
        add4_ordered(accs, sl, tv);
      }
    }
    for (; m < M; ++m) add(icol[(long)m * N], term(m, icol[(long)m * N], gcol[(long)m * N]));
  }
  __syncthreads();
  // rows k of the result: `lines` consecutive columns each
  const int cols = min(lines, N - n0), kn = min(kw, K - w0);
  const int lc = lane & (lines - 1), lk = lane / lines;
  if (lc < cols)
    for (int kk = lk; kk < kn; kk += parts)
      grad_b[((long)batch * K + w0 + kk) * N + n0 + lc] = to_elem<elem_t>(accs[kk * lines + lc]);
}

// Both gradients in one launch, batch item by batch item (ta workgroups of grad_a, then tb of
// grad_b, per item; XCD-aware numbering): both read the item's idx and g, which then come from
// memory once.
template <int PROD>
__global__ __launch_bounds__(64) void k_argmax_bwd_both(const elem_t* __restrict__ amat,
                                                       const elem_t* __restrict__ bmat,
                                                       const float* __restrict__ fac_a,
                                                       const float* __restrict__ fac_b,
                                                       const int32_t* __restrict__ idx,
                                                       const elem_t* __restrict__ g,
                                                       elem_t* __restrict__ grad_a,
                                                       elem_t* __restrict__ grad_b, int M, int K, int N,
                                                       int row_tiles, int kc_a, int ps_a, int vec,
                                                       int col_tiles, int kc_b, int ps_b) {
  __shared__ float accs[kArgAccA > kArgAccB ? kArgAccA : kArgAccB];
  const int ta = row_tiles * kc_a, tb = col_tiles * kc_b;
  const int v = xcd_renumber(blockIdx.x, gridDim.x);
  const int item = v / (ta + tb), r = v - item * (ta + tb);
  if (r < ta)
    argmax_bwd_a_block<PROD>(accs, item * ta + r, bmat, fac_a, idx, g, grad_a, M, K, N, row_tiles, kc_a, ps_a, vec);
  else
    argmax_bwd_b_block<PROD>(accs, item * tb + r - ta, amat, fac_b, idx, g, grad_b, M, K, N, col_tiles, kc_b, ps_b);
}

// Parts per workgroup for a reduction axis of K cells: the smallest power of two that
// covers it (at most 64).
inline int argmax_parts_shift(int K) {
  int ps = 0;
  while (ps < 6 && (kKC << ps) < K) ++ps;
  return ps;
}

template <bool PROD>
int run_argmax_bwd(const elem_t* a, const elem_t* b, const int32_t* idx, const float* factors,
                   const elem_t* g, elem_t* grad_a, elem_t* grad_b, int B, int M, int K, int N,
                   void* stream) {
  if (int e = check_dense_dims(B, M, K, N)) return e;
  const int64_t mk = (int64_t)B * M * K, kn = (int64_t)B * K * N, mn = (int64_t)B * M * N;
  if (missing(idx, mn) || missing(g, mn) || missing(grad_a, mk) || missing(grad_b, kn) ||
      (PROD && !factors && (missing(a, mk) || missing(b, kn))))
    return GENBMM_E_NULLPTR;
  // factors = [a[m, idx] | b[idx, n]], each B*M*N: grad_a needs the second, grad_b the first
  constexpr int kGather = PROD ? 1 : 0;
  hipStream_t s = (hipStream_t)stream;
  if (mk == 0 && kn == 0) return GENBMM_OK;
  // (an empty M or N leaves one gradient without workgroups; the other is then all zeros)
  const int ps_a = argmax_parts_shift(K);
  const int row_tiles = ceil_div(M, 64 >> ps_a), kc_a = ceil_div(K, kKC << ps_a);
  // columns: two parts at most - narrower groups of columns cost more in the strided
  // reads of idx and g than reading them again saves
  const int ps_b = min(argmax_parts_shift(K), 1);
  const int col_tiles = ceil_div(N, 64 >> ps_b), kc_b = ceil_div(K, kKC << ps_b);
  const int64_t total = (int64_t)B * ((int64_t)row_tiles * kc_a + (int64_t)col_tiles * kc_b);
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  const int vec = (N % 4 == 0) && aligned16(idx) && aligned16(g);
  if (PROD && factors)
    hipLaunchKernelGGL((k_argmax_bwd_both<2>), dim3((unsigned)total), dim3(64), 0, s, a, b, factors + mn, factors,
                       idx, g, grad_a, grad_b, M, K, N, row_tiles, kc_a, ps_a, vec && aligned16(factors + mn),
                       col_tiles, kc_b, ps_b);
  else
    hipLaunchKernelGGL((k_argmax_bwd_both<kGather>), dim3((unsigned)total), dim3(64), 0, s, a, b,
                       (const float*)nullptr, (const float*)nullptr, idx, g, grad_a, grad_b, M, K, N, row_tiles,
                       kc_a, ps_a, vec, col_tiles, kc_b, ps_b);
  if (int e = launch_status()) return e;
  return GENBMM_OK;
}

}  // namespace
}  // namespace GENBMM_NS

extern "C" {

// One set per element type: genbmm_argmax_bwd, genbmm_argmax_bwd_f16, ..._bf16, ...
int GENBMM_API(argmax_bwd)(const int32_t* idx, const GENBMM_NS::abi_t* g, GENBMM_NS::abi_t* grad_a,
                           GENBMM_NS::abi_t* grad_b, int B, int M, int K, int N, void* stream) {
  using namespace GENBMM_NS;
  return run_argmax_bwd<false>(nullptr, nullptr, idx, nullptr, el(g), el(grad_a), el(grad_b), B, M, K, N,
                               stream);
}

int GENBMM_API(prodmax_bwd)(const GENBMM_NS::abi_t* a, const GENBMM_NS::abi_t* b, const int32_t* idx,
                            const float* factors, const GENBMM_NS::abi_t* g, GENBMM_NS::abi_t* grad_a,
                            GENBMM_NS::abi_t* grad_b, int B, int M, int K, int N, void* stream) {
  using namespace GENBMM_NS;
  return run_argmax_bwd<true>(el(a), el(b), idx, factors, el(g), el(grad_a), el(grad_b), B, M, K, N,
                              stream);
}

}  // extern "C"
