/*
 * TEST INFRASTRUCTURE ONLY.  Sequential CPU oracle for the genbmm hot path:
 * a plain-C restatement of the reference's per-element arithmetic
 * (matmul_cuda_kernel.cu, banded_cuda_kernel.cu), instantiated for float
 * (orc_f_*) and double (orc_d_*), plus a scalar Philox4x32-10.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * load this; the product (genbmm_amd/) never does.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off -shared -fPIC).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

#define REAL float
#define FN(name) orc_f_##name
#define EXP expf
#define LOG logf
#include "seq_oracle_impl.h"
#undef REAL
#undef FN
#undef EXP
#undef LOG

#define REAL double
#define FN(name) orc_d_##name
#define EXP exp
#define LOG log
#include "seq_oracle_impl.h"
#undef REAL
#undef FN
#undef EXP
#undef LOG

/*
 * Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy
 * as 1, 2, 3", SC'11; Random123 philox.h): per round
 *   hi0:lo0 = M0 * c0,  hi1:lo1 = M1 * c2,
 *   c <- { hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0 },  k0 += W0, k1 += W1.
 */
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* Uniforms of cells first..first+count-1 of stream (seed, offset): cell i takes word
 * i & 3 of Philox(counter = {lo(i >> 2), hi(i >> 2), lo(offset), hi(offset)}, key =
 * {lo(seed), hi(seed)}), top 24 bits scaled by 2^-24. */
void orc_philox_uniform(uint64_t first, uint64_t count, uint64_t seed, uint64_t offset, float* out) {
  for (uint64_t e = 0; e < count; ++e) {
    uint64_t i = first + e;
    uint64_t blk = i >> 2;
    uint32_t ctr[4] = {(uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)offset, (uint32_t)(offset >> 32)};
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t x[4];
    orc_philox4x32_10(ctr, key, x);
    out[e] = (float)(x[i & 3] >> 8) * (1.0f / 16777216.0f);
  }
}
