// Structural operations on band storage (gfx950): pure data movement, bound by
// HBM bandwidth.  data is (batch, n, W = lu + ld + 1) and data[b, c, k] is the
// dense element at row c + k - lu, column c (reference genbmm/sparse.py:12-30).
// The reference builds every one of these from torch cat / flip / unfold /
// diagonal / contiguous calls; here each is one kernel that reads its source once
// and writes its result once, coalesced on both sides (the skewed ones go through
// an LDS tile).
#include "common.h"

namespace GENBMM_NS {
namespace {

constexpr int kST = 256;                 // lanes per workgroup
constexpr int kBlockCells = 8192;        // cells of the result per workgroup (row-granular)
constexpr int kMaxLine = 1 << 20;        // longest row (band width or n) the kernels take
constexpr int kTileBytes = 64 * 1024;    // LDS tile budget of the skewed kernels

typedef float float4_u __attribute__((ext_vector_type(4), aligned(4)));  // any 4-byte address

// i / d for 0 <= i < 2^21 through the float unit (inv = 1/d rounded): (i + 0.5)/d
// is at least 0.5/d away from every integer and the rounding error is below that.
__device__ __forceinline__ int small_div(int i, float inv) {
  return (int)(((float)i + 0.5f) * inv);
}

// ---------------------------------------------------------------- shifts
// out[b, c, k] = in[b, c + dcol, k + dband] where that lies inside (n, w_in), else
// fill.  band_shift(t): dband = t (sparse.py:96-110); band_pad(t): dband = -|t|,
// w_out = w_in + 2|t| (:112-123); band_unshift: dband = -1 (:137-152);
// col_shift(t): dcol = t (:154-165); col_unshift: dcol = -1 (:167-182);
// _expand: dband = -(lu' - lu), wider w_out (:192-197).
__global__ __launch_bounds__(kST) void k_band_shift(const float* __restrict__ in,
                                                   float* __restrict__ out, int n, int w_in,
                                                   int w_out, int dcol, int dband, float fill,
                                                   int rows_per, int chunks, float inv_w) {
  const int batch = blockIdx.x / chunks, chunk = blockIdx.x - batch * chunks;
  const int c0 = chunk * rows_per, rows = min(rows_per, n - c0);
  const float* ib = in + (long)batch * n * w_in;
  float* ob = out + ((long)batch * n + c0) * w_out;
  const int total = rows * w_out;
#pragma unroll 4
  for (int i = threadIdx.x; i < total; i += kST) {
    const int r = small_div(i, inv_w), k = i - r * w_out;
    const int cs = c0 + r + dcol, ks = k + dband;
    const bool ok = cs >= 0 && cs < n && ks >= 0 && ks < w_in;
    const float v = ib[ok ? (long)cs * w_in + ks : 0];
    ob[i] = ok ? v : fill;
  }
}

// ---------------------------------------------------------------- element-wise
// Union band of a and b (lu = max, ld = max); a sits at offset sa, b at sb.
// out = zero everywhere, then a copied in, then op(out, b) on b's cells - the
// reference's three statements (sparse.py:199-212), so cells only a covers hold a
// itself and cells only b covers hold op(zero, b).
enum { kOpAdd = 0, kOpMul = 1, kOpMax = 2, kOpMin = 3 };

__device__ __forceinline__ float apply_op(int op, float x, float y) {
  switch (op) {
    case kOpAdd: return x + y;
    case kOpMul: return x * y;
    case kOpMax: return (x != x || y != y) ? x + y : (x > y ? x : y);  // torch.max propagates NaN
    default: return (x != x || y != y) ? x + y : (x < y ? x : y);
  }
}

__global__ __launch_bounds__(kST) void k_band_op(const float* __restrict__ a,
                                                const float* __restrict__ b,
                                                float* __restrict__ out, int n, int wa, int wb,
                                                int wo, int sa, int sb, int op, float zero,
                                                int rows_per, int chunks, float inv_w) {
  const int batch = blockIdx.x / chunks, chunk = blockIdx.x - batch * chunks;
  const int c0 = chunk * rows_per, rows = min(rows_per, n - c0);
  const float* ab = a + ((long)batch * n + c0) * wa;
  const float* bb = b + ((long)batch * n + c0) * wb;
  float* ob = out + ((long)batch * n + c0) * wo;
  const int total = rows * wo;
#pragma unroll 4
  for (int i = threadIdx.x; i < total; i += kST) {
    const int r = small_div(i, inv_w), k = i - r * wo;
    const int ka = k - sa, kb = k - sb;
    const bool in_a = ka >= 0 && ka < wa, in_b = kb >= 0 && kb < wb;
    const float x = ab[in_a ? r * wa + ka : 0], y = bb[in_b ? r * wb + kb : 0];
    const float base = in_a ? x : zero;
    ob[i] = in_b ? apply_op(op, base, y) : base;
  }
}

// ---------------------------------------------------------------- transpose
// Band of the transposed matrix (lu' = ld, ld' = lu):
//   out[b, c, k] = in[b, c + k - ld, W - 1 - k]   (0 where that row does not exist)
// (reference Transpose / repdiag, sparse.py:33-77, 214-218).  A workgroup owns cb
// result rows; the cb + W - 1 source rows they touch are one contiguous range,
// copied into LDS with an even pitch so that a wave reading along k (address
// stride pitch - 1, odd) meets every bank once.
__global__ __launch_bounds__(kST) void k_band_transpose(const float* __restrict__ in,
                                                       float* __restrict__ out, int n, int W,
                                                       int ld, int cb, int chunks, int pitch,
                                                       float inv_w) {
  extern __shared__ float tile[];
  const int batch = blockIdx.x / chunks, chunk = blockIdx.x - batch * chunks;
  const int c0 = chunk * cb, cols = min(cb, n - c0);
  const float* ib = in + (long)batch * n * W;
  float* ob = out + ((long)batch * n + c0) * W;
  const int first = c0 - ld, src_rows = cols + W - 1;
  // the source rows that exist are one contiguous run of cells: four per lane and load
  const int lo = max(first, 0), hi = min(first + src_rows, n);      // rows [lo, hi)
  const int cells = (hi - lo) * W, skip = (lo - first) * W;
  const float* run = ib + (long)lo * W;
  for (int i = threadIdx.x; i < skip; i += kST) {                   // rows before row 0
    const int r = small_div(i, inv_w);
    tile[r * pitch + (i - r * W)] = 0.f;
  }
  for (int i = skip + cells + threadIdx.x; i < src_rows * W; i += kST) {   // rows past n - 1
    const int r = small_div(i, inv_w);
    tile[r * pitch + (i - r * W)] = 0.f;
  }
#pragma unroll 2
  for (int i = threadIdx.x * 4; i < cells; i += kST * 4) {
    float v[4];
    if (i + 4 <= cells) {
      const float4_u x = *reinterpret_cast<const float4_u*>(run + i);
      v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = run[min(i + j, cells - 1)];
    }
    int r = small_div(skip + i, inv_w), k = skip + i - r * W;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (i + j < cells) tile[r * pitch + k] = v[j];
      if (++k == W) {
        k = 0;
        ++r;
      }
    }
  }
  __syncthreads();
#pragma unroll 4
  for (int i = threadIdx.x; i < cols * W; i += kST) {
    const int c = small_div(i, inv_w), k = i - c * W;
    ob[i] = tile[(c + k) * pitch + (W - 1 - k)];
  }
}

// Bands too wide for the tile: one lane per cell straight from global memory.
__global__ __launch_bounds__(kST) void k_band_transpose_wide(const float* __restrict__ in,
                                                            float* __restrict__ out, int n,
                                                            int W, int ld, long total) {
  const long e = (long)blockIdx.x * kST + threadIdx.x;
  if (e >= total) return;
  const int k = (int)(e % W);
  const long bc = e / W;
  const int c = (int)(bc % n);
  const int src = c + k - ld;
  out[e] = (src >= 0 && src < n) ? in[(bc - c + src) * W + (W - 1 - k)] : 0.f;
}

// ---------------------------------------------------------------- to dense
// out[b, r, c] = data[b, c, r - c + lu] inside the band, else fill
// (sparse.py:184-190).  All but W of the n cells of a row are fill: the kernel
// is a stream of stores, four cells per lane when the rows allow.
template <bool VEC>
__global__ __launch_bounds__(kST) void k_band_to_dense(const float* __restrict__ data,
                                                      float* __restrict__ out, int n, int W,
                                                      int lu, float fill, int rows_per,
                                                      int chunks, float inv_n) {
  const int batch = blockIdx.x / chunks, chunk = blockIdx.x - batch * chunks;
  const int r0 = chunk * rows_per, rows = min(rows_per, n - r0);
  const float* db = data + (long)batch * n * W;
  float* ob = out + ((long)batch * n + r0) * n;
  auto cell = [&](int r, int c) __attribute__((always_inline)) {
    const int k = r - c + lu;
    const bool ok = k >= 0 && k < W;
    const float v = db[ok ? (long)c * W + k : 0];
    return ok ? v : fill;
  };
  if (VEC) {
    const int quads = n >> 2, total = rows * quads;
    const float inv_q = inv_n * 4.f;
  #pragma unroll 4
  for (int i = threadIdx.x; i < total; i += kST) {
      const int rl = small_div(i, inv_q), c = (i - rl * quads) * 4;
      const int r = r0 + rl;
      float4 v = make_float4(fill, fill, fill, fill);
      if (c + 3 >= r - (W - 1 - lu) && c <= r + lu)   // the quad meets the band of row r
        v = make_float4(cell(r, c), cell(r, c + 1), cell(r, c + 2), cell(r, c + 3));
      *reinterpret_cast<float4*>(ob + (long)rl * n + c) = v;
    }
  } else {
    const int total = rows * n;
  #pragma unroll 4
  for (int i = threadIdx.x; i < total; i += kST) {
      const int rl = small_div(i, inv_n), c = i - rl * n;
      ob[i] = cell(r0 + rl, c);
    }
  }
}

// ---------------------------------------------------------------- from dense
// out[b, c, k] = dense[b, c + k - lu, c] (0 where that row does not exist): band
// storage of a dense (n_rows, n) matrix (banddiag, sparse.py:12-30).  A workgroup
// owns cb columns: the (cb + W - 1) x cb block of the dense matrix they touch is
// read row by row into LDS (pitch cb + 1) and written out along k.
__global__ __launch_bounds__(kST) void k_band_from_dense(const float* __restrict__ dense,
                                                        float* __restrict__ out, int n_rows,
                                                        int n, int W, int lu, int cb,
                                                        int cb_shift, int chunks, float inv_w) {
  extern __shared__ float tile[];
  const int batch = blockIdx.x / chunks, chunk = blockIdx.x - batch * chunks;
  const int c0 = chunk * cb, cols = min(cb, n - c0);
  const float* db = dense + (long)batch * n_rows * n;
  float* ob = out + ((long)batch * n + c0) * W;
  const int first = c0 - lu, src_rows = cols + W - 1, pitch = cb + 1;
#pragma unroll 4
  for (int i = threadIdx.x; i < (src_rows << cb_shift); i += kST) {
    const int r = i >> cb_shift, cc = i & (cb - 1);
    const int src = first + r;
    const bool ok = src >= 0 && src < n_rows && cc < cols;
    const float v = db[ok ? (long)src * n + c0 + cc : 0];
    tile[r * pitch + cc] = ok ? v : 0.f;
  }
  __syncthreads();
#pragma unroll 4
  for (int i = threadIdx.x; i < cols * W; i += kST) {
    const int c = small_div(i, inv_w), k = i - c * W;
    ob[i] = tile[(c + k) * pitch + c];
  }
}

__global__ __launch_bounds__(kST) void k_band_from_dense_wide(const float* __restrict__ dense,
                                                             float* __restrict__ out,
                                                             int n_rows, int n, int W, int lu,
                                                             long total) {
  const long e = (long)blockIdx.x * kST + threadIdx.x;
  if (e >= total) return;
  const int k = (int)(e % W);
  const long bc = e / W;
  const int c = (int)(bc % n);
  const long batch = bc / n;
  const int src = c + k - lu;
  out[e] = (src >= 0 && src < n_rows) ? dense[(batch * n_rows + src) * n + c] : 0.f;
}

// ---------------------------------------------------------------- host side
int check_band(int B, int n, int64_t w) {
  if (B < 0 || n < 0) return GENBMM_E_SHAPE;
  if (w < 1) return GENBMM_E_BAND;
  if (w > kMaxLine || n > kMaxLine) return GENBMM_E_SHAPE;
  if ((int64_t)B * n * w > ((int64_t)1 << 40)) return GENBMM_E_SHAPE;
  return GENBMM_OK;
}

// Rows of `line` cells per workgroup and the grid for B * n rows.
int row_blocks(int B, int n, int line, int& rows_per, int& chunks, unsigned& grid) {
  rows_per = kBlockCells / line;
  if (rows_per < 1) rows_per = 1;
  if (rows_per > n) rows_per = n;
  chunks = ceil_div(n, rows_per);
  const int64_t total = (int64_t)B * chunks;
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  grid = (unsigned)total;
  return GENBMM_OK;
}

// Largest power-of-two count of result rows whose LDS tile fits: the more rows, the
// smaller the share of the W - 1 halo rows each workgroup reads on top of its own.
int tile_rows(int W, bool from_dense, int& pitch) {
  for (int cb = from_dense ? 64 : 128; cb >= 8; cb >>= 1) {
    pitch = from_dense ? cb + 1 : W + (W & 1);
    if ((int64_t)(cb + W - 1) * pitch * 4 <= kTileBytes) return cb;
  }
  return 0;
}

int shift_of(int v) {
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}

}  // namespace
}  // namespace GENBMM_NS

extern "C" {

int genbmm_band_shift(const float* data, float* out, int B, int n, int w_in, int w_out, int dcol,
                      int dband, float fill, void* stream) {
  using namespace GENBMM_NS;
  if (int e = check_band(B, n, w_in)) return e;
  if (int e = check_band(B, n, w_out)) return e;
  const int64_t cells = (int64_t)B * n * w_out;
  if (missing(data, (int64_t)B * n * w_in) || missing(out, cells)) return GENBMM_E_NULLPTR;
  if (cells == 0) return GENBMM_OK;
  int rows_per, chunks;
  unsigned grid;
  if (int e = row_blocks(B, n, w_out, rows_per, chunks, grid)) return e;
  hipLaunchKernelGGL(k_band_shift, dim3(grid), dim3(kST), 0, (hipStream_t)stream, data, out, n,
                     w_in, w_out, dcol, dband, fill, rows_per, chunks, 1.0f / (float)w_out);
  return launch_status();
}

int genbmm_band_op(const float* a, int a_lu, int a_ld, const float* b, int b_lu, int b_ld,
                   float* out, int B, int n, int op, float zero, void* stream) {
  using namespace GENBMM_NS;
  if (a_lu < 0 || a_ld < 0 || b_lu < 0 || b_ld < 0) return GENBMM_E_BAND;
  if (op < kOpAdd || op > kOpMin) return GENBMM_E_MODE;
  const int64_t wa = (int64_t)a_lu + a_ld + 1, wb = (int64_t)b_lu + b_ld + 1;
  const int lu = a_lu > b_lu ? a_lu : b_lu, ld = a_ld > b_ld ? a_ld : b_ld;
  const int64_t wo = (int64_t)lu + ld + 1;
  if (int e = check_band(B, n, wo)) return e;
  const int64_t cells = (int64_t)B * n * wo;
  if (missing(a, (int64_t)B * n * wa) || missing(b, (int64_t)B * n * wb) || missing(out, cells))
    return GENBMM_E_NULLPTR;
  if (cells == 0) return GENBMM_OK;
  int rows_per, chunks;
  unsigned grid;
  if (int e = row_blocks(B, n, (int)wo, rows_per, chunks, grid)) return e;
  hipLaunchKernelGGL(k_band_op, dim3(grid), dim3(kST), 0, (hipStream_t)stream, a, b, out, n,
                     (int)wa, (int)wb, (int)wo, lu - a_lu, lu - b_lu, op, zero, rows_per, chunks,
                     1.0f / (float)wo);
  return launch_status();
}

int genbmm_band_transpose(const float* data, float* out, int B, int n, int lu, int ld,
                          void* stream) {
  using namespace GENBMM_NS;
  if (lu < 0 || ld < 0) return GENBMM_E_BAND;
  const int64_t w = (int64_t)lu + ld + 1;
  if (int e = check_band(B, n, w)) return e;
  const int64_t cells = (int64_t)B * n * w;
  if (missing(data, cells) || missing(out, cells)) return GENBMM_E_NULLPTR;
  if (cells == 0) return GENBMM_OK;
  const int W = (int)w;
  int pitch;
  const int cb = tile_rows(W, false, pitch);
  if (cb == 0) {
    const int64_t blocks = (cells + kST - 1) / kST;
    if (blocks > 0x7fffffffLL) return GENBMM_E_SHAPE;
    hipLaunchKernelGGL(k_band_transpose_wide, dim3((unsigned)blocks), dim3(kST), 0,
                       (hipStream_t)stream, data, out, n, W, ld, (long)cells);
    return launch_status();
  }
  const int chunks = ceil_div(n, cb);
  const int64_t total = (int64_t)B * chunks;
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  const size_t lds = (size_t)(cb + W - 1) * pitch * sizeof(float);
  hipLaunchKernelGGL(k_band_transpose, dim3((unsigned)total), dim3(kST), lds,
                     (hipStream_t)stream, data, out, n, W, ld, cb, chunks, pitch,
                     1.0f / (float)W);
  return launch_status();
}

int genbmm_band_to_dense(const float* data, float* out, int B, int n, int lu, int ld, float fill,
                         void* stream) {
  using namespace GENBMM_NS;
  if (lu < 0 || ld < 0) return GENBMM_E_BAND;
  const int64_t w = (int64_t)lu + ld + 1;
  if (int e = check_band(B, n, w)) return e;
  const int64_t cells = (int64_t)B * n * n;
  if (cells > ((int64_t)1 << 40)) return GENBMM_E_SHAPE;
  if (missing(data, (int64_t)B * n * w) || missing(out, cells)) return GENBMM_E_NULLPTR;
  if (cells == 0) return GENBMM_OK;
  int rows_per, chunks;
  unsigned grid;
  if (int e = row_blocks(B, n, n, rows_per, chunks, grid)) return e;
  const float inv_n = 1.0f / (float)n;
  if (n % 4 == 0 && aligned16(out))
    hipLaunchKernelGGL((k_band_to_dense<true>), dim3(grid), dim3(kST), 0, (hipStream_t)stream,
                       data, out, n, (int)w, lu, fill, rows_per, chunks, inv_n);
  else
    hipLaunchKernelGGL((k_band_to_dense<false>), dim3(grid), dim3(kST), 0, (hipStream_t)stream,
                       data, out, n, (int)w, lu, fill, rows_per, chunks, inv_n);
  return launch_status();
}

int genbmm_band_from_dense(const float* dense, float* out, int B, int n_rows, int n, int lu,
                           int ld, void* stream) {
  using namespace GENBMM_NS;
  if (lu < 0 || ld < 0) return GENBMM_E_BAND;
  if (n_rows < 0 || n_rows > kMaxLine) return GENBMM_E_SHAPE;
  const int64_t w = (int64_t)lu + ld + 1;
  if (int e = check_band(B, n, w)) return e;
  const int64_t cells = (int64_t)B * n * w, src = (int64_t)B * n_rows * n;
  if (src > ((int64_t)1 << 40)) return GENBMM_E_SHAPE;
  if (missing(out, cells) || (missing(dense, src) && n_rows > 0)) return GENBMM_E_NULLPTR;
  if (cells == 0) return GENBMM_OK;
  const int W = (int)w;
  int pitch;
  const int cb = n_rows > 0 ? tile_rows(W, true, pitch) : 0;
  if (cb == 0) {
    const int64_t blocks = (cells + kST - 1) / kST;
    if (blocks > 0x7fffffffLL) return GENBMM_E_SHAPE;
    hipLaunchKernelGGL(k_band_from_dense_wide, dim3((unsigned)blocks), dim3(kST), 0,
                       (hipStream_t)stream, dense, out, n_rows, n, W, lu, (long)cells);
    return launch_status();
  }
  const int chunks = ceil_div(n, cb);
  const int64_t total = (int64_t)B * chunks;
  if (total > 0x7fffffffLL) return GENBMM_E_SHAPE;
  const size_t lds = (size_t)(cb + W - 1) * pitch * sizeof(float);
  hipLaunchKernelGGL(k_band_from_dense, dim3((unsigned)total), dim3(kST), lds,
                     (hipStream_t)stream, dense, out, n_rows, n, W, lu, cb, shift_of(cb), chunks,
                     1.0f / (float)W);
  return launch_status();
}

}  // extern "C"
