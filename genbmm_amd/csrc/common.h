// Shared device/host helpers for the gfx950 semiring-matmul kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/genbmm_gfx950.h"

// Element type of the caller's tensors.  The dense sources are compiled once per element
// type (GENBMM_ELEM: 0 float, 1 IEEE binary16, 2 bfloat16), each into a namespace and a
// set of entry-point names of its own; arithmetic, LDS and every workspace are fp32 in all
// three: a half value is widened by the load that fetches it and a result is rounded
// (to nearest even) by the store that writes it.
#ifndef GENBMM_ELEM
#define GENBMM_ELEM 0
#endif
#if GENBMM_ELEM == 0
#define GENBMM_NS genbmm_f32
#define GENBMM_API(name) genbmm_##name
#elif GENBMM_ELEM == 1
#define GENBMM_NS genbmm_f16
#define GENBMM_API(name) genbmm_##name##_f16
#elif GENBMM_ELEM == 2
#define GENBMM_NS genbmm_bf16
#define GENBMM_API(name) genbmm_##name##_bf16
#else
#error "GENBMM_ELEM: 0 (float), 1 (binary16) or 2 (bfloat16)"
#endif

namespace GENBMM_NS {

#if GENBMM_ELEM == 0
typedef float elem_t;
typedef float abi_t;       // what the C header declares for an element
#elif GENBMM_ELEM == 1
typedef _Float16 elem_t;
typedef uint16_t abi_t;
#else
typedef __bf16 elem_t;
typedef uint16_t abi_t;
#endif
constexpr bool kElemF32 = GENBMM_ELEM == 0;
inline const elem_t* el(const abi_t* p) { return reinterpret_cast<const elem_t*>(p); }
inline elem_t* el(abi_t* p) { return reinterpret_cast<elem_t*>(p); }

// Floor of every running maximum, as in the reference kernels
// (matmul_cuda_kernel.cu:31,62,93,139; banded_cuda_kernel.cu:44,79).
constexpr float kFloor = -1e9f;
constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;

// v_exp_f32 / v_log_f32: base-2 hardware transcendentals.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// exp(x) for x that is already a difference (x <= ~0): one multiply + v_exp_f32.
__device__ __forceinline__ float fast_exp(float x) { return fast_exp2(x * kLog2e); }

constexpr int kPad = 4;  // LDS row padding (floats); keeps float4 alignment

// ------------------------------------------------------- four elements at a time
// ld4 / st4: element alignment only (the hardware takes misaligned dwordx4 / dwordx2;
// rows of odd-sized matrices start anywhere).  ld4a / st4a: the address is a multiple of
// four elements.  The masked forms touch the first cnt (<= 0: none, >= 4: all) elements.
typedef float f4v __attribute__((ext_vector_type(4)));
typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));
typedef _Float16 h4v __attribute__((ext_vector_type(4)));
typedef _Float16 h4u __attribute__((ext_vector_type(4), aligned(2)));
typedef __bf16 b4v __attribute__((ext_vector_type(4)));
typedef __bf16 b4u __attribute__((ext_vector_type(4), aligned(2)));
__device__ __forceinline__ float4 from_f4v(f4v f) { return make_float4(f.x, f.y, f.z, f.w); }
// A result is rounded to fp32 first and to the half type second, exactly as if the float
// kernel's output were converted afterwards.  Left alone, the compiler folds a multiply that
// feeds the conversion into one instruction with a single rounding (v_fma_mixlo_f16), which
// differs on ties; `settled` hides the value's origin from it (no instruction is emitted).
__device__ __forceinline__ float settled(float x) {
  asm volatile("" : "+v"(x));
  return x;
}
__device__ __forceinline__ f4v to_f4v(float4 v) {
  f4v f;
  f.x = settled(v.x); f.y = settled(v.y); f.z = settled(v.z); f.w = settled(v.w);
  return f;
}
// float -> element, for scalar stores
template <class E>
__device__ __forceinline__ E to_elem(float x) {
  if constexpr (sizeof(E) == 4) return x;
  else return (E)settled(x);
}
__device__ __forceinline__ float4 ld4(const float* p) {
  const float4u v = *reinterpret_cast<const float4u*>(p);
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float4 ld4(const _Float16* p) {
  return from_f4v(__builtin_convertvector(*reinterpret_cast<const h4u*>(p), f4v));
}
__device__ __forceinline__ float4 ld4(const __bf16* p) {
  return from_f4v(__builtin_convertvector(*reinterpret_cast<const b4u*>(p), f4v));
}
__device__ __forceinline__ float4 ld4a(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ld4a(const _Float16* p) {
  return from_f4v(__builtin_convertvector(*reinterpret_cast<const h4v*>(p), f4v));
}
__device__ __forceinline__ float4 ld4a(const __bf16* p) {
  return from_f4v(__builtin_convertvector(*reinterpret_cast<const b4v*>(p), f4v));
}
__device__ __forceinline__ void st4(float* p, float4 v) {
  float4u u;
  u.x = v.x; u.y = v.y; u.z = v.z; u.w = v.w;
  *reinterpret_cast<float4u*>(p) = u;
}
__device__ __forceinline__ void st4(_Float16* p, float4 v) {
  *reinterpret_cast<h4u*>(p) = __builtin_convertvector(to_f4v(v), h4u);
}
__device__ __forceinline__ void st4(__bf16* p, float4 v) {
  *reinterpret_cast<b4u*>(p) = __builtin_convertvector(to_f4v(v), b4u);
}
__device__ __forceinline__ void st4a(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void st4a(_Float16* p, float4 v) {
  *reinterpret_cast<h4v*>(p) = __builtin_convertvector(to_f4v(v), h4v);
}
__device__ __forceinline__ void st4a(__bf16* p, float4 v) {
  *reinterpret_cast<b4v*>(p) = __builtin_convertvector(to_f4v(v), b4v);
}
template <class E>
__device__ __forceinline__ float4 ld4m(const E* p, int cnt, float fill) {
  if (cnt >= 4) return ld4(p);
  float4 r = make_float4(fill, fill, fill, fill);
  if (cnt > 0) r.x = p[0];
  if (cnt > 1) r.y = p[1];
  if (cnt > 2) r.z = p[2];
  return r;
}
template <class E>
__device__ __forceinline__ void st4m(E* p, int cnt, float4 v) {
  if (cnt >= 4) {
    st4(p, v);
    return;
  }
  if (cnt > 0) p[0] = to_elem<E>(v.x);
  if (cnt > 1) p[1] = to_elem<E>(v.y);
  if (cnt > 2) p[2] = to_elem<E>(v.z);
}
__device__ __forceinline__ int clamp4(int x) { return min(max(x, 0), 4); }

// ---------------------------------------------------------------- tile loaders
//
// Both loaders move a [RED x OUT] tile into LDS laid out as lds[red][out]
// (row stride OUT + kPad) through registers, so that the global loads of the
// next tile can be in flight while the current tile is being consumed.
// Out-of-range elements are filled with 0; kernels never let those reach a
// stored result (reduction loops stop at the true extent, stores are masked).

// Operand stored in global memory as [out][red] (contiguous along the
// reduction axis), leading dimension ld.
template <int OUT, int RED, int NT>
struct TileOutMajor {
  static constexpr int C4 = RED / 4;
  static constexpr int NV = OUT * C4;
  static constexpr int PER = (NV + NT - 1) / NT;
  static constexpr int LD = OUT + kPad;
  float4 r[PER];

  template <class E>
  __device__ __forceinline__ void gload(const E* __restrict__ base, long ld,
                                        int out0, int red0, int out_lim,
                                        int red_lim, bool vec, int tid) {
#pragma unroll
    for (int l = 0; l < PER; ++l) {
      const int idx = tid + l * NT;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (NV % NT == 0 || idx < NV) {
        const int row = idx / C4, c4 = idx % C4;
        const int go = out0 + row, gr = red0 + c4 * 4;
        if (go < out_lim && gr < red_lim) {
          const E* p = base + (long)go * ld + gr;
          if (vec && gr + 3 < red_lim) {
            v = ld4a(p);
          } else {
            v.x = p[0];
            if (gr + 1 < red_lim) v.y = p[1];
            if (gr + 2 < red_lim) v.z = p[2];
            if (gr + 3 < red_lim) v.w = p[3];
          }
        }
      }
      r[l] = v;
    }
  }

  __device__ __forceinline__ void sstore(float* __restrict__ lds, int tid) const {
#pragma unroll
    for (int l = 0; l < PER; ++l) {
      const int idx = tid + l * NT;
      if (NV % NT == 0 || idx < NV) {
        const int row = idx / C4, c4 = idx % C4;
        float* p = lds + (c4 * 4) * LD + row;
        p[0] = r[l].x;
        p[LD] = r[l].y;
        p[2 * LD] = r[l].z;
        p[3 * LD] = r[l].w;
      }
    }
  }
};

// Operand stored in global memory as [red][out] (contiguous along the output
// axis), leading dimension ld.
template <int OUT, int RED, int NT>
struct TileRedMajor {
  static constexpr int C4 = OUT / 4;
  static constexpr int NV = RED * C4;
  static constexpr int PER = (NV + NT - 1) / NT;
  static constexpr int LD = OUT + kPad;
  float4 r[PER];

  template <class E>
  __device__ __forceinline__ void gload(const E* __restrict__ base, long ld,
                                        int out0, int red0, int out_lim,
                                        int red_lim, bool vec, int tid) {
#pragma unroll
    for (int l = 0; l < PER; ++l) {
      const int idx = tid + l * NT;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (NV % NT == 0 || idx < NV) {
        const int row = idx / C4, c4 = idx % C4;
        const int gr = red0 + row, go = out0 + c4 * 4;
        if (gr < red_lim && go < out_lim) {
          const E* p = base + (long)gr * ld + go;
          if (vec && go + 3 < out_lim) {
            v = ld4a(p);
          } else {
            v.x = p[0];
            if (go + 1 < out_lim) v.y = p[1];
            if (go + 2 < out_lim) v.z = p[2];
            if (go + 3 < out_lim) v.w = p[3];
          }
        }
      }
      r[l] = v;
    }
  }

  __device__ __forceinline__ void sstore(float* __restrict__ lds, int tid) const {
#pragma unroll
    for (int l = 0; l < PER; ++l) {
      const int idx = tid + l * NT;
      if (NV % NT == 0 || idx < NV) {
        const int row = idx / C4, c4 = idx % C4;
        *reinterpret_cast<float4*>(lds + row * LD + c4 * 4) = r[l];
      }
    }
  }
};

// Read NV4 float4 fragments lds[off + q*stride4 .. +4) into dst[4*NV4].
template <int NV4>
__device__ __forceinline__ void lds_frag(const float* __restrict__ row, int off,
                                         int stride, float* dst) {
#pragma unroll
  for (int q = 0; q < NV4; ++q) {
    const float4 v = *reinterpret_cast<const float4*>(row + off + q * stride);
    dst[4 * q + 0] = v.x;
    dst[4 * q + 1] = v.y;
    dst[4 * q + 2] = v.z;
    dst[4 * q + 3] = v.w;
  }
}

// 16-byte alignment test used to enable four-element global accesses (stricter than
// needed for the half types).
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ------------------------------------------------------------------- Philox
// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3",
// SC'11): multipliers 0xD2511F53 / 0xCD9E8D57, Weyl key increments
// 0x9E3779B9 / 0xBB67AE85, ten rounds.
struct Philox4 {
  uint32_t x[4];
};

__host__ __device__ inline Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2,
                                                 uint32_t c3, uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    const uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  Philox4 r;
  r.x[0] = c0; r.x[1] = c1; r.x[2] = c2; r.x[3] = c3;
  return r;
}

// One Philox block serves four consecutive output cells: cell i takes word i & 3 of
// Philox(counter = {lo(i >> 2), hi(i >> 2), lo(offset), hi(offset)}, key = seed); its
// top 24 bits scaled by 2^-24 are the uniform in [0,1).  (The 64-bit products of the
// ten rounds are the cost of a draw: a lane that owns four adjacent cells pays once.)
__host__ __device__ inline Philox4 philox_block(uint64_t block, uint64_t seed, uint64_t offset) {
  return philox4x32_10((uint32_t)block, (uint32_t)(block >> 32), (uint32_t)offset,
                       (uint32_t)(offset >> 32), (uint32_t)seed, (uint32_t)(seed >> 32));
}
__host__ __device__ inline float philox_scale(uint32_t word) {
  return (float)(word >> 8) * (1.0f / 16777216.0f);
}
// Uniform in [0,1) of output cell `i` for stream (seed, offset).
__host__ __device__ inline float philox_uniform(uint64_t i, uint64_t seed, uint64_t offset) {
  const Philox4 r = philox_block(i >> 2, seed, offset);
  const uint32_t w = (i & 2) ? ((i & 1) ? r.x[3] : r.x[2]) : ((i & 1) ? r.x[1] : r.x[0]);
  return philox_scale(w);
}

// Uniforms of the four consecutive cells i .. i+3.  aligned: i is a multiple of four
// (one block); otherwise the cells straddle two blocks.
__host__ __device__ inline void philox_uniform4(uint64_t i, bool aligned, uint64_t seed,
                                                uint64_t offset, float (&u)[4]) {
  const Philox4 r0 = philox_block(i >> 2, seed, offset);
  if (aligned) {
    u[0] = philox_scale(r0.x[0]); u[1] = philox_scale(r0.x[1]);
    u[2] = philox_scale(r0.x[2]); u[3] = philox_scale(r0.x[3]);
    return;
  }
  const Philox4 r1 = philox_block((i >> 2) + 1, seed, offset);
  const uint32_t w[8] = {r0.x[0], r0.x[1], r0.x[2], r0.x[3], r1.x[0], r1.x[1], r1.x[2], r1.x[3]};
  const int s = (int)(i & 3);
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    uint32_t v = w[q];
#pragma unroll
    for (int t = 1; t < 4; ++t) v = s == t ? w[q + t] : v;
    u[q] = philox_scale(v);
  }
}

// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.
// Renumber them so that every XCD works on one contiguous run of tiles (the
// tiles of a batch item share their operands): XCD x takes n / 8 of them, one
// more if x < n % 8, and workgroup w is the (w / 8)-th of XCD w % 8.
__device__ __forceinline__ int xcd_renumber(int w, int n) {
  const int q = n >> 3, r = n & 7, x = w & 7;
  return x * q + min(x, r) + (w >> 3);
}
// Four ordered additions with one LDS round trip: the four cells are read together,
// the sums are chained in registers (a cell that was already hit earlier in the group
// takes that sum instead of what it read), and written back in order.  A term whose k
// is not this lane's goes to the lane's spare cell.
__device__ __forceinline__ void add4_ordered(float* __restrict__ accs, const int (&s)[4],
                                             const float (&v)[4]) {
  const float r0 = accs[s[0]], r1 = accs[s[1]], r2 = accs[s[2]], r3 = accs[s[3]];
  const float v0 = __fadd_rn(r0, v[0]);
  const float v1 = __fadd_rn(s[1] == s[0] ? v0 : r1, v[1]);
  const float v2 = __fadd_rn(s[2] == s[1] ? v1 : (s[2] == s[0] ? v0 : r2), v[2]);
  const float v3 = __fadd_rn(s[3] == s[2] ? v2 : (s[3] == s[1] ? v1 : (s[3] == s[0] ? v0 : r3)), v[3]);
  accs[s[0]] = v0;
  accs[s[1]] = v1;
  accs[s[2]] = v2;
  accs[s[3]] = v3;
}

// ------------------------------------------------------------- host helpers
inline int check_dense_dims(int B, int M, int K, int N) {
  if (B < 0 || M < 0 || K < 0 || N < 0) return GENBMM_E_SHAPE;
  // element counts are 64-bit inside; 2^37 elements (half a terabyte of floats) is beyond
  // any device buffer and keeps one-lane-per-cell grids (cells / 256) within 32 bits
  const int64_t lim = (int64_t)1 << 37;
  if ((int64_t)B * M * K > lim || (int64_t)B * K * N > lim || (int64_t)B * M * N > lim)
    return GENBMM_E_SHAPE;
  // launch grids: one workgroup per tile of 32 x 32 at the smallest, two tile lists in one
  // launch at the most - a grid beyond 2^31 - 1 workgroups would wrap silently
  const int64_t grid_lim = (int64_t)1 << 30;
  auto tiles = [](int64_t batch, int x, int y) { return batch * ((x + 31) / 32) * ((y + 31) / 32); };
  if (tiles(B, M, N) > grid_lim || tiles(B, M, K) > grid_lim || tiles(B, K, N) > grid_lim)
    return GENBMM_E_SHAPE;
  return GENBMM_OK;
}

// A pointer may be NULL only if the buffer it names has no elements.
inline bool missing(const void* p, int64_t count) { return p == nullptr && count > 0; }

inline int launch_status() {
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? GENBMM_OK : (int)e;
}

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

}  // namespace GENBMM_NS
