// Backward of the banded max product as two scatters: every output cell (i, j)
// hands its incoming gradient to the one a-cell and the one b-cell its argmax
// names, so the work is one pass over g and idx (n * Wo cells per batch item)
// instead of one pass per gradient cell.
//
//   grad_a[i, k]  += g[i, j]   for k  = idx[i, j],                 j ascending
//   grad_b[o, k2] += g[i, j]   for k2 = idx[i, j] - j + Wb - 1,    i ascending
//                                    (o = i + j - r_lu, i.e. j descending)
//
// which are the reference's summation orders (banded_cuda_kernel.cu:104-152 and
// the transposed call of sparse.py:625-635), so the sums come out bit for bit.
// One workgroup per strip of 64 rows; a lane owns a row of the gradient and walks
// its cells in that order, accumulating in LDS at [k][lane]: whatever k each of the 64
// lanes adds to, the lanes stay in 64 different banks (with the rows 65 apart a wave's
// additions met at random: 11.6 M conflict cycles per launch at 64 x 4096, 65 diagonals).
// For the row-wise write-out the sums change places once, through registers, to [row][k]
// with an odd row length.  g and idx pass through LDS tiles of 32 diagonals so that global
// memory is read in runs along the band.
// Cells outside the matrix carry index 0 from the forward and are masked here.
#pragma once

#include "banded_cells.h"

namespace GENBMM_NS {

constexpr int kAT = 64;        // rows per strip
constexpr int kAJ = 32;        // diagonals per tile
constexpr int kAC = kAJ + 1;   // tile row stride
constexpr int kAS = kAT;       // accumulators: [k][lane]

// accumulators [W][64], one spare cell per lane (terms that are not the lane's), tiles
__host__ __device__ inline int argmax_acc_floats(int W) { return kAT * W + 256; }
inline size_t argmax_bwd_a_bytes(int Wa) { return sizeof(float) * ((size_t)argmax_acc_floats(Wa) + 2 * kAT * kAC); }
inline size_t argmax_bwd_b_bytes(int Wb) {
  return sizeof(float) * ((size_t)argmax_acc_floats(Wb) + 2 * (kAT + kAJ - 1) * kAC);
}

// The sums leave as rows, 32 cells of the band at a time: [k][lane] -> `tile` as [row][33]
// (a wave moving one k for 64 rows meets 64 banks on both sides) -> memory in runs along the
// band.  tile: kAT * kAC floats (the g tile, no longer needed).
__device__ __forceinline__ void argmax_write_out(const float* __restrict__ acc, float* __restrict__ tile, int W,
                                                 elem_t* __restrict__ out, int rows, int tid) {
  const int lane = tid & 63, wave = tid >> 6;
  for (int kc = 0; kc < W; kc += kAJ) {
    __syncthreads();  // the sums are complete / the previous chunk has left the tile
#pragma unroll
    for (int q = 0; q < kAJ / 4; ++q) {
      const int kk = wave + 4 * q;
      if (kc + kk < W) tile[lane * kAC + kk] = acc[(kc + kk) * kAS + lane];
    }
    __syncthreads();
    for (int e = tid; e < kAT * kAJ; e += 256) {
      const int r = e >> 5, c = e & 31;
      if (r < rows && kc + c < W) out[(long)r * W + kc + c] = to_elem<elem_t>(tile[r * kAC + c]);
    }
  }
}

// Tile of ROWS x 32 cells of g and idx: load() starts the global reads (masked
// cells read nothing), store() puts them into LDS - the next tile is in flight
// while the current one is consumed.
template <int ROWS>
struct ArgTile {
  static constexpr int PER = (ROWS * kAJ + 255) / 256;
  float gv[PER];
  int iv[PER];
  // row0: g row of tile row 0; the cell (row0 + r, jc + c) counts if its row is in
  // [0, n), j < Wo and, for need_o, its o = i + j - r_lu is in [0, n); for skew (a tile
  // whose rows of b run along its diagonals) only if it lies on the diagonal of one of the
  // strip's 64 rows - the corners of the tile are not read
  __device__ __forceinline__ void load(const elem_t* __restrict__ gb, const int32_t* __restrict__ ib,
                                       int row0, int jc, int n, int Wo, int r_lu, bool need_o,
                                       bool skew, int tid) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = tid + 256 * u, r = e >> 5, c = e & 31;
      const int i = row0 + r, j = jc + c, o = i + j - r_lu;
      const bool ok = r < ROWS && i >= 0 && i < n && j < Wo && (!need_o || (o >= 0 && o < n)) &&
                      (!skew || (unsigned)(r - (kAJ - 1) + c) < (unsigned)kAT);
      gv[u] = ok ? gb[(long)i * Wo + j] : 0.f;
      iv[u] = ok ? ib[(long)i * Wo + j] : -1;
    }
  }
  __device__ __forceinline__ void store(float* __restrict__ gt, int* __restrict__ it, int tid) const {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = tid + 256 * u, r = e >> 5, c = e & 31;
      if (r < ROWS) {
        gt[r * kAC + c] = gv[u];
        it[r * kAC + c] = iv[u];
      }
    }
  }
};

// Four waves per strip: all walk the same cells in the same order, wave w adds
// only the cells whose target index is w mod 4, so the per-target order is kept
// and the dependent read-modify-write chains are a quarter as long; the additions
// go four at a time through add4_ordered (one LDS round trip for four cells).
__global__ __launch_bounds__(256) void k_band_argmax_bwd_a(const BandArgs p, int strips) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int n = p.n, Wa = p.Wa, Wo = p.Wo;
  float* acc = smem;                                      // [Wa][65] + 256 spare cells
  float* gt = acc + argmax_acc_floats(Wa);                // [64][33]
  int* it = reinterpret_cast<int*>(gt + kAT * kAC);       // [64][33]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int batch = blockIdx.x / strips, i0 = (blockIdx.x - batch * strips) * kAT;
  const long bn = (long)batch * n;
  const elem_t* gb = p.g + bn * Wo;
  const int32_t* ib = p.idx + bn * Wo;
  for (int e = tid; e < argmax_acc_floats(Wa); e += 256) acc[e] = 0.f;
  const int spare = argmax_acc_floats(Wa) - 256 + tid;
  ArgTile<kAT> tile;
  tile.load(gb, ib, i0, 0, n, Wo, p.r_lu, true, false, tid);
  for (int jc = 0; jc < Wo; jc += kAJ) {
    __syncthreads();
    tile.store(gt, it, tid);
    __syncthreads();
    if (jc + kAJ < Wo) tile.load(gb, ib, i0, jc + kAJ, n, Wo, p.r_lu, true, false, tid);
#pragma unroll 2
    for (int c = 0; c < kAJ; c += 4) {
      int sl[4];
      float tv[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int k = it[lane * kAC + c + q];
        sl[q] = (k >= 0 && k < Wa && (k & 3) == wave) ? k * kAS + lane : spare;
        tv[q] = gt[lane * kAC + c + q];
      }
      add4_ordered(acc, sl, tv);
    }
  }
  argmax_write_out(acc, gt, Wa, p.o0 + (bn + i0) * Wa, min(kAT, n - i0), tid);
}

__global__ __launch_bounds__(256) void k_band_argmax_bwd_b(const BandArgs p, int strips) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  constexpr int kRows = kAT + kAJ - 1;  // 95 rows of g / idx feed 64 rows of b per tile
  const int n = p.n, Wb = p.Wb, Wo = p.Wo;
  float* acc = smem;                                      // [Wb][65] + 256 spare cells
  float* gt = acc + argmax_acc_floats(Wb);                // [95][33]
  int* it = reinterpret_cast<int*>(gt + kRows * kAC);     // [95][33]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int batch = blockIdx.x / strips, o0 = (blockIdx.x - batch * strips) * kAT;
  const long bn = (long)batch * n;
  const elem_t* gb = p.g + bn * Wo;
  const int32_t* ib = p.idx + bn * Wo;
  for (int e = tid; e < argmax_acc_floats(Wb); e += 256) acc[e] = 0.f;
  const int spare = argmax_acc_floats(Wb) - 256 + tid;
  // i = o + r_lu - j ascends as j descends: last tile first, columns right to left;
  // tile row 0 holds g row o0 + r_lu - jc - 31
  const int jlast = ((Wo - 1) / kAJ) * kAJ;
  auto row0_of = [&](int jc) { return o0 + p.r_lu - jc - (kAJ - 1); };
  ArgTile<kRows> tile;
  tile.load(gb, ib, row0_of(jlast), jlast, n, Wo, p.r_lu, false, true, tid);
  for (int jc = jlast; jc >= 0; jc -= kAJ) {
    __syncthreads();
    tile.store(gt, it, tid);
    __syncthreads();
    if (jc > 0) tile.load(gb, ib, row0_of(jc - kAJ), jc - kAJ, n, Wo, p.r_lu, false, true, tid);
    if (o0 + lane < n) {
#pragma unroll 2
      for (int c4 = kAJ - 1; c4 >= 0; c4 -= 4) {
        int sl[4];
        float tv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          // cell (i, j) with i + j - r_lu = o0 + lane sits in tile row lane + 31 - c
          const int c = c4 - q, r = lane + (kAJ - 1) - c;
          const int k = it[r * kAC + c];
          const int k2 = k - (jc + c) + Wb - 1;
          sl[q] = (k >= 0 && k2 >= 0 && k2 < Wb && (k2 & 3) == wave) ? k2 * kAS + lane : spare;
          tv[q] = gt[r * kAC + c];
        }
        add4_ordered(acc, sl, tv);
      }
    }
  }
  argmax_write_out(acc, gt, Wb, p.o1 + (bn + o0) * Wb, min(kAT, n - o0), tid);
}

}  // namespace GENBMM_NS
