// What genbmm_logbmm_fwd leaves in its workspace for other entry points of the
// library (the sampling sweep reads the factors instead of taking exponentials again).
#pragma once

#include "common.h"

namespace GENBMM_NS {

// First word of the workspace's header: which forward filled the workspace last.
constexpr int kWsNone = 0;  // one that leaves no per-tile flags (exact and whole-item kernels)
constexpr int kWsMfma = 1;  // the matrix-core forward: flags, EA, EB and 1/S
constexpr int kWsFast = 2;  // the factored vector-ALU forward: flags only
constexpr int kWsSelf = 3;  // the one-tile-per-item forward: the maxima only

struct LogFactors {
  const float* ea;   // exp(a - row maximum), (B, M, K)
  const float* eb;   // exp(b - column maximum), (B, K, N)
  float* scratch;    // (B, M, N): 1/S after the forward; free for the caller to overwrite
  int* valid;        // the workspace's "factors present" word; clear it when scratch is overwritten
};

// genbmm_logbmm_fwd, except that shapes whose forward would keep nothing but the maxima
// take the kernels that leave the factors (what log_fwd_writes_factors() describes).
int log_fwd_with_factors(const elem_t* a, const elem_t* b, elem_t* out, float* stats, int B, int M, int K,
                         int N, hipStream_t s);

// True (and *f filled) if a log_fwd_with_factors call with this workspace and these sizes
// writes the factors: the same decision the forward takes, made on the host.
bool log_fwd_writes_factors(const float* stats, int B, int M, int K, int N, LogFactors* f);

// For a workspace that log_fwd_writes_factors() accepts: the sampling sweep on the
// matrix cores.  Leaves in idx the code -2 - group (groups of 16 terms; K - 1, final: the
// prefix sums never reach the target) and in the scratch array rem at the start of that
// group; tiles that the forward or the sweep flagged are redone exactly (out and the
// final index).  The caller resolves the codes.
bool log_sample_mfma_ok(int K);  // the sweep below takes reductions up to 126 slabs of 16 terms
int log_sample_sweep_mfma(const elem_t* a, const elem_t* b, elem_t* out, int32_t* idx,
                          const float* stats, uint64_t seed, uint64_t offset, int B, int M, int K,
                          int N, hipStream_t s);

// samplebmm on a problem whose forward cuts its reduction into pieces (few result tiles, a long
// K): log_sample_cut_ok() tells whether this is one; log_sample_cut() runs that forward - out, the
// maxima and every piece's sum stay in the workspace - and draws every cell's index from the sums:
// the piece in which the prefix passes the cell's target, then the terms of that one piece.
bool log_sample_cut_ok(const float* stats, int B, int M, int K, int N);
int64_t log_sample_cut_floats(int B, int M, int K, int N);  // workspace floats behind the header (0: no cut)
int log_sample_cut(const elem_t* a, const elem_t* b, elem_t* out, int32_t* idx, float* stats, uint64_t seed,
                   uint64_t offset, int B, int M, int K, int N, hipStream_t s);

}  // namespace GENBMM_NS
