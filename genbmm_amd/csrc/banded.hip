// Banded-matrix semiring multiply: forward, backward (both operands) and the
// log-semiring second-order terms (gfx950).
//
// Band storage (reference genbmm/sparse.py:12-30): data[b, c, k] is the dense
// element (row c + k - lu, column c); row c of `data` is dense column c.
// For operands a (lu=a_lu, ld=a_ld, width Wa) and b (b_lu, b_ld, Wb) the
// product has lu = a_lu + b_ld, ld = a_ld + b_lu, width Wo = Wa + Wb - 1 and
//
//   out[i, j] = (+)_k a[i, k] (x) b[o, k2],   o  = i + j - lu_out,
//                                            k2 = k - j + (Wb - 1),
//
// over the k with 0 <= k < Wa, 0 <= k2 < Wb and 0 <= i + k - a_lu < n
// (reference banded_cuda_kernel.cu:32-51; k2 there is (pos - o) + b_lu with
// pos = i + k - a_lu, which simplifies to the expression above).  k2 does not
// depend on i, so for a fixed output diagonal j the operands are walked as
// two straight runs: a[i, klo..khi] and b[o, klo-j+Wb-1 ..].
//
// One lane per output element with lanes along the band axis (the contiguous
// axis of every tensor), so stores are coalesced and neighbouring lanes read
// overlapping runs that the vector L1 / L2 serve.
#include <type_traits>

#include "banded_argmax.h"
#include "banded_block.h"
#include "banded_direct.h"
#include "banded_flat.h"
#include "banded_max.h"
#include "banded_sample.h"
#include "banded_strip.h"

namespace GENBMM_NS {
namespace {

constexpr size_t kStripLdsLimit = 64 * 1024;  // dynamic LDS available without opting in

// Workspace of the log product: EA (B*n*Wa), EB (B*n*Wb), alpha (B*n), beta (B*n),
// R (B*n*Wo) floats from the forward, and H (B*n*Wo) that the backward fills.
inline bool dir_bwd_ok(const BandArgs& p);
// (H only where the backward is not the memory-fed one, which forms it on the fly)
inline size_t band_ws_floats(const BandArgs& p, int B) {
  return (size_t)B * p.n * ((size_t)p.Wa + p.Wb + (dir_bwd_ok(p) ? 1 : 2) * (size_t)p.Wo + 2);
}
// Which bands the strip kernels take (forward / backward): tiles within 64 KB of
// LDS, the sliding tile large enough to double as the output staging tiles.
inline bool fwd_strip_ok(const BandArgs& p) {
  const StripDims sd = strip_dims(p.Wa, p.Wb);
  const bool tiles_fit = (size_t)kBR * sd.ld_sl >= (size_t)2 * kBT * kBC;
  return tiles_fit && sd.ld_own <= 256 && sd.ld_sl <= 256 && sd.bytes <= kStripLdsLimit;
}
inline bool bwd_strip_ok(const BandArgs& p) {
  if (p.Wa > 8 * 4 * kMaxKB || p.Wb > 8 * 4 * kMaxKB) return false;
  const StripDims da = strip_dims(p.Wa, p.Wb), db = strip_dims(p.Wb, p.Wa);
  return max(bwd_strip_bytes(da, true), bwd_strip_bytes(db, true)) <= kStripLdsLimit &&
         max(max(da.ld_own, da.ld_sl), max(db.ld_own, db.ld_sl)) <= 128;
}
constexpr size_t kMmLdsLimit = 80 * 1024;  // two workgroups' tiles in a compute unit's LDS
// The memory-fed kernels (banded_direct.h): a plan within their limits, offsets inside a
// batch item within 32 bits.
inline bool dir_ok(int kind, const BandArgs& p, int min_w) {
  DirPlan plan;
  return min(p.Wa, p.Wb) >= min_w && (long)p.n * p.Wo < (1L << 30) &&
         dir_plan(plan, kind, p.a_lu, p.Wa, p.b_lu, p.Wb);
}
// From 3 diagonals on, except the forward of the plain product, which one lane per cell does
// faster below 7 (measured at 64 x 4096, memory-fed against what it replaces: 3 diagonals plain
// forward 0.020 ms against 0.009, backward 0.044 against 0.074, log forward with its
// preparation 0.043 against 0.011 without a workspace, log backward 0.060 against 0.219; 7
// diagonals plain forward 0.020 against 0.023).
constexpr int kDirMinW = 3, kDirMinWPlainFwd = 7;
inline bool dir_fwd_ok(const BandArgs& p, int min_w = kDirMinW) { return dir_ok(kDirFwd, p, min_w); }
inline bool dir_bwd_ok(const BandArgs& p) {
  return dir_ok(kDirGradA, p, kDirMinW) && dir_ok(kDirGradB, p, kDirMinW);
}
// The workspace of the log product is filled and used only when both directions have a
// kernel that works on it (memory-fed or strip), so that forward and backward always agree
// on whether it holds anything.
inline bool workspace_used(const BandArgs& p) {
  const bool fwd = dir_fwd_ok(p) ||
                   (fwd_strip_ok(p) &&
                    strip_dims(p.Wa, p.Wb).bytes + sizeof(float) * (kBT + p.Wo + kBJ) <= kStripLdsLimit);
  return fwd && (dir_bwd_ok(p) || bwd_strip_ok(p));
}

inline bool prep_fwd(const BandArgs& p, int mode, const float* workspace) {
  return mode == GENBMM_BAND_LOG && workspace != nullptr && workspace_used(p);
}

// The whole-strip max-plus forward: from 8 diagonals on (measured at 64 x 4096: 9 diagonals
// 0.035 ms against 0.042, 17: 0.046 against 0.126, 65: 0.29 against 0.36; 5: 0.031 against
// 0.015 for one lane per cell), bands whose tiles fit two workgroups per compute unit.
// Diagonals per workgroup: the whole result while it has at most 160 diagonals and its tiles
// fit two workgroups per compute unit; otherwise the widest segment (a multiple of 8) whose
// tiles fit - two workgroups per compute unit if possible, else one.  0: none fits.
inline int max_fwd_segment(const BandArgs& p) {
  if (min(p.Wa, p.Wb) < 8) return 0;
  if (p.Wo <= 160 && max_dims(p.Wa, p.Wb, p.Wo).bytes <= kMmLdsLimit) return p.Wo;
  // just past that the chunked strip kernel is the faster one (81 diagonals per operand at
  // 16 x 4096: 0.14 ms against 0.23 in two segments); segments take over where it ends
  if (fwd_strip_ok(p)) return 0;
  for (size_t limit : {kMmLdsLimit, (size_t)160 * 1024})
    for (int w = min(160, p.Wo & ~7); w >= 16; w -= 8)
      if (max_dims(p.Wa, p.Wb, w).bytes <= limit) return w;
  return 0;
}
inline bool max_fwd_ok(const BandArgs& p) { return max_fwd_segment(p) > 0; }
inline void launch_max_fwd(const BandArgs& p, int B, hipStream_t s) {
  const int Wseg = max_fwd_segment(p), nseg = ceil_div(p.Wo, Wseg);
  const MaxDims d = max_dims(p.Wa, p.Wb, Wseg);
  const int strips = ceil_div(p.n, kMaxRows);
  if (d.bytes > kStripLdsLimit)
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k_band_max_fwd),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)d.bytes);
  const long rows = (long)B * p.n;
  hipLaunchKernelGGL(k_band_max_fwd, dim3((unsigned)((long)B * strips * nseg)), dim3(256), d.bytes, s, p, strips, d,
                     rows * p.Wa, rows * p.Wb, nseg, Wseg);
}

inline void launch_prep(const BandArgs& p, const elem_t* a, int a_lu, const elem_t* b, int b_lu, int B,
                        hipStream_t s) {
  const long rows = (long)B * p.n;
  const PrepSide pa{a, p.ws_ea, p.ws_al, p.Wa, a_lu, odd(p.Wa)}, pb{b, p.ws_eb, p.ws_be, p.Wb, b_lu, odd(p.Wb)};
  const int blocks_a = (int)((rows + kPrepRows - 1) / kPrepRows), blocks_b = blocks_a;
  const size_t lds = sizeof(float) * (size_t)kPrepRows * max(pa.ld, pb.ld);
  const int vec = aligned16(a) && aligned16(b) && aligned16(p.ws_ea) && aligned16(p.ws_eb);
  if (lds > kStripLdsLimit)
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k_band_prep), hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds);
  hipLaunchKernelGGL(k_band_prep, dim3((unsigned)(blocks_a + blocks_b)), dim3(256), lds, s, pa, pb, p.n, rows,
                     blocks_a, vec);
}

// The block kernel (banded_block.h) takes the forward where it is the faster one: from about 53
// diagonals per operand (measured at 64 x 4096, block against memory-fed: 49 diagonals 0.067 ms
// against 0.063, 57: 0.078 against 0.084, 65: 0.083 against 0.098; log product with its
// preparation 0.145 / 0.138, 0.165 / 0.177, 0.193 / 0.214) up to where its staged blocks still fit
// a compute unit's LDS (65 diagonals per operand; 73 do not).
constexpr int kBlkMinW = 53;
inline bool blk_fwd_ok(const BandArgs& p, int B) {
  BlkPlan g;
  return min(p.Wa, p.Wb) >= kBlkMinW && (long)p.n * p.Wo < (1L << 30) && blk_plan_fwd(g, p.Wa, p.Wb, p.n, B, 8);
}
template <bool PREP>
inline void launch_blk_fwd(const BandArgs& p, int B, hipStream_t s) {
  BlkPlan g;
  blk_plan_fwd(g, p.Wa, p.Wb, p.n, B, 8);
  const int nblocks = B * g.chunks;
  const size_t lds = blk_lds_bytes(g);
  auto go = [&](auto kern, int sw) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(64 * (g.ncw + sw)), lds, s, p, g, nblocks, (long)B * p.n);
  };
  if (max(g.NSa, g.NSb) <= 6) go(k_band_blk_fwd<PREP, 4, 3, 3>, 4);
  else go(k_band_blk_fwd<PREP, 4, 4, 4>, 4);
}

template <int KIND, bool PREP>
inline void launch_dir(const BandArgs& p, int B, hipStream_t s) {
  const int blocks = ceil_div(p.n, 16 * kDirWaves);
  const int nblocks = B * blocks;
  DirPlan plan;
  dir_plan(plan, KIND, p.a_lu, p.Wa, p.b_lu, p.Wb);
  const int wave_lds = dir_wave_lds(plan, KIND, PREP);
  auto go = [&](auto kern, const auto& table) {
    if ((size_t)kDirWaves * wave_lds > kStripLdsLimit)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                kDirWaves * wave_lds);
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(64 * kDirWaves), kDirWaves * wave_lds, s, p, table,
                       blocks, nblocks, (long)B * p.n, wave_lds);
  };
  if (plan.steps <= kDirStepsSmall) go(k_band_dir<KIND, PREP, DirPlanSmall>, dir_plan_small(plan));
  else go(k_band_dir<KIND, PREP, DirPlan>, plan);
}

// grad_a and grad_b in one launch where both plans travel in the small form, else one launch each.
template <bool PREP>
inline void launch_dir_grads(const BandArgs& p, int B, hipStream_t s) {
  DirPlan pa, pb;
  dir_plan(pa, kDirGradA, p.a_lu, p.Wa, p.b_lu, p.Wb);
  dir_plan(pb, kDirGradB, p.a_lu, p.Wa, p.b_lu, p.Wb);
  if (pa.steps > kDirStepsSmall || pb.steps > kDirStepsSmall) {
    launch_dir<kDirGradA, PREP>(p, B, s);
    launch_dir<kDirGradB, PREP>(p, B, s);
    return;
  }
  const int blocks = ceil_div(p.n, 16 * kDirWaves);
  const int nblocks = B * blocks;
  const int wave_lds = max(dir_wave_lds(pa, kDirGradA, PREP), dir_wave_lds(pb, kDirGradB, PREP));
  auto kern = k_band_dir_grads<PREP, DirPlanSmall>;
  if ((size_t)kDirWaves * wave_lds > kStripLdsLimit)
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              kDirWaves * wave_lds);
  hipLaunchKernelGGL(kern, dim3(2u * (unsigned)nblocks), dim3(64 * kDirWaves), kDirWaves * wave_lds, s, p,
                     dir_plan_small(pa), dir_plan_small(pb), blocks, nblocks, (long)B * p.n, wave_lds);
}

inline void set_workspace(BandArgs& p, float* ws, int B) {
  const size_t rows = (size_t)B * p.n;
  p.ws_ea = ws;
  p.ws_eb = p.ws_ea + rows * p.Wa;
  p.ws_al = p.ws_eb + rows * p.Wb;
  p.ws_be = p.ws_al + rows;
  p.ws_r = p.ws_be + rows;
  p.ws_h = dir_bwd_ok(p) ? nullptr : p.ws_r + rows * p.Wo;
}

}  // namespace
}  // namespace GENBMM_NS

extern "C" {

#if GENBMM_ELEM == 0  // sizes do not depend on the element type: every workspace is float
size_t genbmm_banded_workspace_size(int a_lu, int a_ld, int b_lu, int b_ld, int B, int n) {
  using namespace GENBMM_NS;
  BandArgs p{};
  if (fill_band(p, a_lu, a_ld, b_lu, b_ld, B, n)) return 0;
  return band_ws_floats(p, B);
}

int genbmm_banded_on_matrix_cores(int a_lu, int a_ld, int b_lu, int b_ld, int B, int n) {
  using namespace GENBMM_NS;
  BandArgs p{};
  if (fill_band(p, a_lu, a_ld, b_lu, b_ld, B, n)) return 0;
  return workspace_used(p) ? 1 : 0;
}

size_t genbmm_banded_scratch_size(int a_lu, int a_ld, int b_lu, int b_ld, int B, int n) {
  using namespace GENBMM_NS;
  BandArgs p{};
  if (fill_band(p, a_lu, a_ld, b_lu, b_ld, B, n)) return 0;
  return dir_bwd_ok(p) || !workspace_used(p) ? 0 : (size_t)B * n * p.Wo;
}
#endif

int GENBMM_API(banded_fwd)(const GENBMM_NS::abi_t* a_, int a_lu, int a_ld, const GENBMM_NS::abi_t* b_, int b_lu,
                           int b_ld, GENBMM_NS::abi_t* out_, int32_t* idx, float* workspace, int B, int n, int mode,
                           void* stream) {
  using namespace GENBMM_NS;
  const elem_t* a = el(a_);
  const elem_t* b = el(b_);
  elem_t* out = el(out_);
  if (mode != GENBMM_BAND_LOG && mode != GENBMM_BAND_MAX && mode != GENBMM_BAND_MUL)
    return GENBMM_E_MODE;
  BandArgs p{};
  if (int e = fill_band(p, a_lu, a_ld, b_lu, b_ld, B, n)) return e;
  if ((int64_t)B * n == 0) return GENBMM_OK;
  if (!a || !b || !out || (mode == GENBMM_BAND_MAX && !idx)) return GENBMM_E_NULLPTR;
  p.a = a; p.b = b; p.o0 = out; p.oidx = idx;
  const long total = (long)B * n * p.Wo;
  if (total == 0) return GENBMM_OK;
  hipStream_t s = (hipStream_t)stream;
  const StripDims sd = strip_dims(p.Wa, p.Wb);
  const bool dir = dir_fwd_ok(p, mode == GENBMM_BAND_MUL ? kDirMinWPlainFwd : kDirMinW);
  if (dir && (mode == GENBMM_BAND_MUL || prep_fwd(p, mode, workspace))) {
    const bool blk = blk_fwd_ok(p, B);
    if (mode == GENBMM_BAND_LOG) {
      set_workspace(p, workspace, B);
      launch_prep(p, a, a_lu, b, b_lu, B, s);
      if (blk) launch_blk_fwd<true>(p, B, s);
      else launch_dir<kDirFwd, true>(p, B, s);
    } else {
      if (blk) launch_blk_fwd<false>(p, B, s);
      else launch_dir<kDirFwd, false>(p, B, s);
    }
    return launch_status();
  }
  if (mode == GENBMM_BAND_MAX && max_fwd_ok(p)) {
    launch_max_fwd(p, B, s);
    return launch_status();
  }
  if (fwd_strip_ok(p)) {
    const int strips = ceil_div(n, kBT);
    const dim3 grid((unsigned)((long)B * strips));
    const int nq = ceil_div(max(sd.ld_own, sd.ld_sl), 64);
    // the prepared log product also stages beta for every row its outputs can meet
    const size_t lds = sd.bytes + (prep_fwd(p, mode, workspace) ? sizeof(float) * (kBT + p.Wo + kBJ) : 0);
    auto go = [&](auto kern) {
      hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, p, strips, sd.ld_own, sd.ld_sl);
    };
    const bool prep = prep_fwd(p, mode, workspace);
    if (prep) {  // EA, alpha and EB, beta once, instead of per strip and chunk
      set_workspace(p, workspace, B);
      launch_prep(p, a, a_lu, b, b_lu, B, s);
    }
    auto pick = [&](auto nqc) {
      constexpr int Q = decltype(nqc)::value;
      if (prep) go(k_band_fwd_strip<kSemLogPrep, Q>);
      else if (mode == GENBMM_BAND_LOG) go(k_band_fwd_strip<kSemLog, Q>);
      else if (mode == GENBMM_BAND_MAX) go(k_band_fwd_strip<kSemMax, Q>);
      else go(k_band_fwd_strip<kSemMul, Q>);
    };
    if (nq <= 1) pick(std::integral_constant<int, 1>{});
    else if (nq == 2) pick(std::integral_constant<int, 2>{});
    else pick(std::integral_constant<int, 4>{});
    return launch_status();
  }
  if (mode == GENBMM_BAND_LOG)
    hipLaunchKernelGGL((k_band_fwd<GENBMM_BAND_LOG, elem_t>), blocks_for(total), dim3(256), 0, s, p, total);
  else if (mode == GENBMM_BAND_MAX)
    hipLaunchKernelGGL((k_band_fwd<GENBMM_BAND_MAX, elem_t>), blocks_for(total), dim3(256), 0, s, p, total);
  else
    hipLaunchKernelGGL((k_band_fwd<GENBMM_BAND_MUL, elem_t>), blocks_for(total), dim3(256), 0, s, p, total);
  return launch_status();
}

int GENBMM_API(banded_sample_fwd)(const GENBMM_NS::abi_t* a_, int a_lu, int a_ld, const GENBMM_NS::abi_t* b_,
                                  int b_lu, int b_ld, GENBMM_NS::abi_t* out_, int32_t* idx, float* workspace,
                                  uint64_t seed, uint64_t offset, int B, int n, void* stream) {
  using namespace GENBMM_NS;
  const elem_t* a = el(a_);
  const elem_t* b = el(b_);
  elem_t* out = el(out_);
  BandArgs p{};
  if (int e = fill_band(p, a_lu, a_ld, b_lu, b_ld, B, n)) return e;
  if ((int64_t)B * n == 0) return GENBMM_OK;
  if (!a || !b || !out || !idx) return GENBMM_E_NULLPTR;
  // out: the log product, on the workspace where there is one
  if (int e = GENBMM_API(banded_fwd)(a_, a_lu, a_ld, b_, b_lu, b_ld, out_, nullptr, workspace, B, n, GENBMM_BAND_LOG,
                                     stream))
    return e;
  p.a = a; p.b = b; p.out = out; p.oidx = idx;
  const long total = (long)B * n * p.Wo;
  hipStream_t s = (hipStream_t)stream;
  const bool dir = dir_fwd_ok(p, kDirMinW);
  const bool prepared = prep_fwd(p, GENBMM_BAND_LOG, workspace) && (dir || fwd_strip_ok(p));
  const int Wseg = max_fwd_segment(p);
  if (prepared && Wseg > 0) {
    set_workspace(p, workspace, B);
    const int nseg = ceil_div(p.Wo, Wseg), strips = ceil_div(p.n, kMaxRows);
    const MaxDims d = max_dims(p.Wa, p.Wb, Wseg);
    if ((long)B * strips * nseg > 0x7fffffffL) return GENBMM_E_SHAPE;
    hipLaunchKernelGGL(k_band_sample_targets, blocks_for((total + 3) / 4), dim3(256), 0, s, p.ws_r, idx, total, seed,
                       offset);
    if (d.bytes > kStripLdsLimit)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k_band_sample_fwd<elem_t>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)d.bytes);
    const long rows = (long)B * p.n;
    hipLaunchKernelGGL(k_band_sample_fwd<elem_t>, dim3((unsigned)((long)B * strips * nseg)), dim3(256), d.bytes, s, p,
                       strips, d, rows * p.Wa, rows * p.Wb, nseg, Wseg, seed, offset);
    return launch_status();
  }
  hipLaunchKernelGGL(k_band_sample_cells<elem_t>, blocks_for(total), dim3(256), 0, s, p, total, seed, offset);
  return launch_status();
}

namespace GENBMM_NS {
namespace {
// `scratch`: where g / S goes in the prepared log product; NULL: the workspace's own part
static int banded_bwd(const elem_t* a, int a_lu, int a_ld, const elem_t* b, int b_lu, int b_ld,
               const elem_t* out, const int32_t* idx, float* workspace, float* scratch, const elem_t* g,
               elem_t* grad_a, elem_t* grad_b, int B, int n, int mode, void* stream) {
  if (mode == GENBMM_BAND_SAMPLE) mode = GENBMM_BAND_MAX;  // a drawn index scatters like an arg-max
  if (mode != GENBMM_BAND_LOG && mode != GENBMM_BAND_MAX && mode != GENBMM_BAND_MUL)
    return GENBMM_E_MODE;
  BandArgs p{};
  if (int e = fill_band(p, a_lu, a_ld, b_lu, b_ld, B, n)) return e;
  if ((int64_t)B * n == 0) return GENBMM_OK;
  if (!a || !b || !g || !grad_a || !grad_b || (mode == GENBMM_BAND_LOG && !out) ||
      (mode == GENBMM_BAND_MAX && !idx))
    return GENBMM_E_NULLPTR;
  p.a = a; p.b = b; p.out = out; p.idx = idx; p.g = g; p.o0 = grad_a; p.o1 = grad_b;
  const long ta = (long)B * n * p.Wa, tb = (long)B * n * p.Wb;
  if (ta == 0) return GENBMM_OK;
  hipStream_t s = (hipStream_t)stream;
  if (mode != GENBMM_BAND_MAX && (mode == GENBMM_BAND_MUL || (workspace && workspace_used(p))) && dir_bwd_ok(p)) {
    if (mode == GENBMM_BAND_MUL) {
      launch_dir_grads<false>(p, B, s);
    } else {  // H = g / S is formed by both kernels as they read g: the workspace is only read
      set_workspace(p, workspace, B);
      launch_dir_grads<true>(p, B, s);
    }
    return launch_status();
  }
  if (mode != GENBMM_BAND_MAX && bwd_strip_ok(p)) {
    const bool lg = mode == GENBMM_BAND_LOG;
    const StripDims da = strip_dims(p.Wa, p.Wb), db = strip_dims(p.Wb, p.Wa);
    const size_t na = bwd_strip_bytes(da, lg), nb = bwd_strip_bytes(db, lg);
    {
      const int strips = ceil_div(n, kBT);
      const dim3 grid((unsigned)((long)B * strips));
      const int nq = ceil_div(max(max(da.ld_own, da.ld_sl), max(db.ld_own, db.ld_sl)), 64);
      // on the forward's workspace: a (+,x) backward plus epilogue.  H = g / S needs a place: the
      // caller's scratch, or the workspace's own part - which exists exactly for the bands whose
      // backward is not the memory-fed one (band_ws_floats); without one, the kernels below
      // rebuild the weights from `out`
      if (lg && workspace && workspace_used(p) && (scratch || !dir_bwd_ok(p))) {
        set_workspace(p, workspace, B);
        if (scratch) p.ws_h = scratch;
        // H = g * R once for both gradients (NaN marks a cell whose R is not usable)
        const long cells = (long)B * n * p.Wo;
        hipLaunchKernelGGL(k_band_h, dim3((unsigned)min((cells + 1023) / 1024, (long)0x7fffffff)),
                           dim3(256), 0, s, g, p.ws_r, p.ws_h, cells);
        if (nq <= 1) {
          hipLaunchKernelGGL((k_band_bwd_strip<false, true, 1, true>), grid, dim3(256), na, s, p, strips, da.ld_own, da.ld_sl, bwd_sl_floats(da));
          hipLaunchKernelGGL((k_band_bwd_strip<false, false, 1, true>), grid, dim3(256), nb, s, p, strips, db.ld_own, db.ld_sl, bwd_sl_floats(db));
        } else {
          hipLaunchKernelGGL((k_band_bwd_strip<false, true, 2, true>), grid, dim3(256), na, s, p, strips, da.ld_own, da.ld_sl, bwd_sl_floats(da));
          hipLaunchKernelGGL((k_band_bwd_strip<false, false, 2, true>), grid, dim3(256), nb, s, p, strips, db.ld_own, db.ld_sl, bwd_sl_floats(db));
        }
        return launch_status();
      }
      if (nq <= 1) {
        if (lg) {
          hipLaunchKernelGGL((k_band_bwd_strip<true, true, 1>), grid, dim3(256), na, s, p, strips, da.ld_own, da.ld_sl, bwd_sl_floats(da));
          hipLaunchKernelGGL((k_band_bwd_strip<true, false, 1>), grid, dim3(256), nb, s, p, strips, db.ld_own, db.ld_sl, bwd_sl_floats(db));
        } else {
          hipLaunchKernelGGL((k_band_bwd_strip<false, true, 1>), grid, dim3(256), na, s, p, strips, da.ld_own, da.ld_sl, bwd_sl_floats(da));
          hipLaunchKernelGGL((k_band_bwd_strip<false, false, 1>), grid, dim3(256), nb, s, p, strips, db.ld_own, db.ld_sl, bwd_sl_floats(db));
        }
      } else {
        if (lg) {
          hipLaunchKernelGGL((k_band_bwd_strip<true, true, 2>), grid, dim3(256), na, s, p, strips, da.ld_own, da.ld_sl, bwd_sl_floats(da));
          hipLaunchKernelGGL((k_band_bwd_strip<true, false, 2>), grid, dim3(256), nb, s, p, strips, db.ld_own, db.ld_sl, bwd_sl_floats(db));
        } else {
          hipLaunchKernelGGL((k_band_bwd_strip<false, true, 2>), grid, dim3(256), na, s, p, strips, da.ld_own, da.ld_sl, bwd_sl_floats(da));
          hipLaunchKernelGGL((k_band_bwd_strip<false, false, 2>), grid, dim3(256), nb, s, p, strips, db.ld_own, db.ld_sl, bwd_sl_floats(db));
        }
      }
      return launch_status();
    }
  }
  if (mode == GENBMM_BAND_MAX &&
      max(argmax_bwd_a_bytes(p.Wa), argmax_bwd_b_bytes(p.Wb)) <= kDirLdsLimit) {  // a compute unit's LDS
    const int strips = ceil_div(n, kAT);
    const dim3 grid((unsigned)((long)B * strips));
    const size_t na = argmax_bwd_a_bytes(p.Wa), nb = argmax_bwd_b_bytes(p.Wb);
    if (na > kStripLdsLimit)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k_band_argmax_bwd_a),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)na);
    if (nb > kStripLdsLimit)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(k_band_argmax_bwd_b),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)nb);
    hipLaunchKernelGGL(k_band_argmax_bwd_a, grid, dim3(256), na, s, p, strips);
    hipLaunchKernelGGL(k_band_argmax_bwd_b, grid, dim3(256), nb, s, p, strips);
    return launch_status();
  }
  if (mode == GENBMM_BAND_LOG) {
    hipLaunchKernelGGL((k_band_bwd_a<GENBMM_BAND_LOG, elem_t>), blocks_for(ta), dim3(256), 0, s, p, ta);
    hipLaunchKernelGGL((k_band_bwd_b<GENBMM_BAND_LOG, elem_t>), blocks_for(tb), dim3(256), 0, s, p, tb);
  } else if (mode == GENBMM_BAND_MAX) {
    hipLaunchKernelGGL((k_band_bwd_a<GENBMM_BAND_MAX, elem_t>), blocks_for(ta), dim3(256), 0, s, p, ta);
    hipLaunchKernelGGL((k_band_bwd_b<GENBMM_BAND_MAX, elem_t>), blocks_for(tb), dim3(256), 0, s, p, tb);
  } else {
    hipLaunchKernelGGL((k_band_bwd_a<GENBMM_BAND_MUL, elem_t>), blocks_for(ta), dim3(256), 0, s, p, ta);
    hipLaunchKernelGGL((k_band_bwd_b<GENBMM_BAND_MUL, elem_t>), blocks_for(tb), dim3(256), 0, s, p, tb);
  }
  return launch_status();
}
}  // namespace
}  // namespace GENBMM_NS

int GENBMM_API(banded_bwd)(const GENBMM_NS::abi_t* a, int a_lu, int a_ld, const GENBMM_NS::abi_t* b, int b_lu,
                           int b_ld, const GENBMM_NS::abi_t* out, const int32_t* idx, float* workspace,
                           const GENBMM_NS::abi_t* g, GENBMM_NS::abi_t* grad_a, GENBMM_NS::abi_t* grad_b, int B, int n,
                           int mode, void* stream) {
  using namespace GENBMM_NS;
  return banded_bwd(el(a), a_lu, a_ld, el(b), b_lu, b_ld, el(out), idx, workspace, nullptr, el(g), el(grad_a),
                    el(grad_b), B, n, mode, stream);
}

int GENBMM_API(banded_bwd_scratch)(const GENBMM_NS::abi_t* a, int a_lu, int a_ld, const GENBMM_NS::abi_t* b,
                                   int b_lu, int b_ld, const GENBMM_NS::abi_t* out, const int32_t* idx,
                                   const float* workspace, float* scratch, const GENBMM_NS::abi_t* g,
                                   GENBMM_NS::abi_t* grad_a, GENBMM_NS::abi_t* grad_b, int B, int n, int mode,
                                   void* stream) {
  using namespace GENBMM_NS;
  if (workspace && !scratch && mode == GENBMM_BAND_LOG &&
      genbmm_banded_scratch_size(a_lu, a_ld, b_lu, b_ld, B, n) != 0)
    return GENBMM_E_NULLPTR;
  return banded_bwd(el(a), a_lu, a_ld, el(b), b_lu, b_ld, el(out), idx, const_cast<float*>(workspace), scratch,
                    el(g), el(grad_a), el(grad_b), B, n, mode, stream);
}


// `t_scratch`: B * n * Wo floats for the half element types, where t (the gradient with respect
// to g, which the other two gradients read back) must stay unrounded; the float build keeps it in
// grad_g itself and takes no such argument.
#if GENBMM_ELEM == 0
int genbmm_banded_bwdbwd(const float* a, int a_lu, int a_ld, const float* b, int b_lu, int b_ld,
                         const float* out, const float* g, const float* u_a, const float* u_b,
                         float* grad_a, float* grad_b, float* grad_g, int B, int n,
                         void* stream) {
  float* t_scratch = grad_g;
#else
int GENBMM_API(banded_bwdbwd)(const GENBMM_NS::abi_t* a_, int a_lu, int a_ld, const GENBMM_NS::abi_t* b_, int b_lu,
                              int b_ld, const GENBMM_NS::abi_t* out_, const GENBMM_NS::abi_t* g_,
                              const GENBMM_NS::abi_t* ua_, const GENBMM_NS::abi_t* ub_, GENBMM_NS::abi_t* ga_,
                              GENBMM_NS::abi_t* gb_, GENBMM_NS::abi_t* gg_, float* t_scratch, int B, int n,
                              void* stream) {
  using GENBMM_NS::el;
  const GENBMM_NS::elem_t *a = el(a_), *b = el(b_), *out = el(out_), *g = el(g_), *u_a = el(ua_), *u_b = el(ub_);
  GENBMM_NS::elem_t *grad_a = el(ga_), *grad_b = el(gb_), *grad_g = el(gg_);
#endif
  using namespace GENBMM_NS;
  BandArgs p{};
  if (int e = fill_band(p, a_lu, a_ld, b_lu, b_ld, B, n)) return e;
  if ((int64_t)B * n == 0) return GENBMM_OK;
  if (!a || !b || !out || !g || !grad_a || !grad_b || !grad_g || !t_scratch || (!u_a && !u_b))
    return GENBMM_E_NULLPTR;
  p.a = a; p.b = b; p.out = out; p.g = g; p.ua = u_a; p.ub = u_b;
  p.o0 = grad_a; p.o1 = grad_b; p.o2 = grad_g;
  const long ta = (long)B * n * p.Wa, tb = (long)B * n * p.Wb, to = (long)B * n * p.Wo;
  if (to == 0) return GENBMM_OK;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(k_band_bb_t<elem_t>, blocks_for(to), dim3(256), 0, s, p, t_scratch, to);
  hipLaunchKernelGGL(k_band_bb_a<elem_t>, blocks_for(ta), dim3(256), 0, s, p, t_scratch, ta);
  hipLaunchKernelGGL(k_band_bb_b<elem_t>, blocks_for(tb), dim3(256), 0, s, p, t_scratch, tb);
  return launch_status();
}

#if GENBMM_ELEM == 0
const char* genbmm_version(void) { return "genbmm-gfx950 0.1"; }

const char* genbmm_error_string(int code) {
  switch (code) {
    case GENBMM_OK: return "ok";
    case GENBMM_E_NULLPTR: return "a required pointer argument is NULL";
    case GENBMM_E_SHAPE: return "a dimension is negative or too large";
    case GENBMM_E_MODE: return "unknown semiring mode or kernel path";
    case GENBMM_E_BAND: return "negative band width";
    case GENBMM_E_TOOBIG: return "problem exceeds the fixed workspace of this entry point";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
  }
}
#endif

}  // extern "C"
