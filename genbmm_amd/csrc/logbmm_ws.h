// What genbmm_logbmm_fwd leaves in its workspace for other entry points of the
// library (the sampling sweep reads the factors instead of taking exponentials again).
#pragma once

namespace genbmm {

struct LogFactors {
  const float* ea;   // exp(a - row maximum), (B, M, K)
  const float* eb;   // exp(b - column maximum), (B, K, N)
  float* scratch;    // (B, M, N): 1/S after the forward; free for the caller to overwrite
  int* valid;        // the workspace's "factors present" word; clear it when scratch is overwritten
};

// True (and *f filled) if a genbmm_logbmm_fwd call with this workspace and these sizes
// writes the factors: the same decision the forward takes, made on the host.
bool log_fwd_writes_factors(const float* stats, int B, int M, int K, int N, LogFactors* f);

}  // namespace genbmm
