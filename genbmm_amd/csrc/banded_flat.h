// Shared by the banded kernels that stage operand rows in LDS as they lie in memory:
// the 16-byte vector type and the flat copy of a run of band rows.
#pragma once

#include <cfloat>
#include <cstdint>

#include "banded_strip.h"

namespace GENBMM_NS {

constexpr int kMmSlack = 8;    // spare floats around a staged block
typedef float mm_f4 __attribute__((ext_vector_type(4)));

// `count` elements starting at tensor[first] - rows of W elements - read in pieces of four
// elements (16 bytes of floats, 8 of a half type) from the aligned address below and laid
// down as floats with row stride `pitch`: tensor[first + r * W + k] lands at
// L[origin() + r * pitch + k].
// load() only issues the reads of one batch of 256 * U pieces, store() consumes them.
// E: float (a workspace) or the element type of the caller's tensors (widened by the load).
template <int U, class E = float>
struct MmFlat {
  mm_f4 v[U];
  int nvec, lead, W, gap;
  unsigned magic;  // ceil(2^32 / W)
  const E* abeg;
  bool inside;     // every piece lies inside the tensor

  // [tensor, tensor_end): the whole tensor; a piece that crosses its ends is read element by element
  __device__ __forceinline__ void init(const E* tensor, const E* tensor_end, long first, int count,
                                       int W_, int pitch) {
    const E* beg = tensor + first;
    lead = (int)((reinterpret_cast<uintptr_t>(beg) & (4 * sizeof(E) - 1)) / sizeof(E));
    abeg = beg - lead;
    nvec = count > 0 ? (lead + count + 3) >> 2 : 0;
    W = W_;
    gap = pitch - W_;
    magic = (unsigned)((0x100000000ull + (unsigned)W - 1) / (unsigned)W);
    inside = abeg >= tensor && abeg + 4 * (long)nvec <= tensor_end;
  }
  __device__ __forceinline__ int origin() const { return lead + gap; }
  __device__ __forceinline__ bool more(int batch) const { return batch * 256 * U < nvec; }
  __device__ __forceinline__ void load(const E* lo, const E* hi, int batch, int tid) {
    if (inside) {  // uniform
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int vi = tid + 256 * (u + batch * U);
        v[u] = mm_f4{0.f, 0.f, 0.f, 0.f};
        if (vi < nvec) {
          const float4 x = ld4a(abeg + 4 * vi);
          v[u] = mm_f4{x.x, x.y, x.z, x.w};
        }
      }
      return;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int vi = tid + 256 * (u + batch * U);
      mm_f4 x = mm_f4{0.f, 0.f, 0.f, 0.f};
      if (vi < nvec) {
        const E* q = abeg + 4 * vi;
        for (int t = 0; t < 4; ++t)
          if (q + t >= lo && q + t < hi) x[t] = q[t];
      }
      v[u] = x;
    }
  }
  // returns whether this thread saw a value that is not finite.  Piece v holds the flat
  // cells 4 v - lead ...; with u = 4 v + W - lead, its first cell is in row u / W - 1
  // (row -1: the cells before the first wanted one), and W >= 4 lets it cross into one
  // more row at most.
  __device__ __forceinline__ bool store(float* __restrict__ L, int batch, int tid) const {
    bool bad = false;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int vi = tid + 256 * (u + batch * U);
      if (vi < nvec) {
        const mm_f4 x = v[u];
        bad |= !(fabsf(x[0]) <= FLT_MAX) || !(fabsf(x[1]) <= FLT_MAX) || !(fabsf(x[2]) <= FLT_MAX) ||
               !(fabsf(x[3]) <= FLT_MAX);
        const int f = 4 * vi, uu = f + W - lead;
        const int r1 = (int)__umulhi((unsigned)uu, magic), k = uu - r1 * W;
        float* at = L + (f + r1 * gap);
        const int nb = W - k;  // cells of the piece before its row ends, at least one
        at[0] = x[0];
#pragma unroll
        for (int t = 1; t < 4; ++t) at[t + (t >= nb ? gap : 0)] = x[t];
      }
    }
    return bad;
  }
};

}  // namespace GENBMM_NS
