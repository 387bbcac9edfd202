"""genbmm_logbmm_fwd_static: the logbmm forward on the library's own fixed workspace, for
callers that cannot allocate.  Called through the C ABI and compared with
genbmm_logbmm_fwd on a caller-allocated workspace (same kernels: equal bit for bit, and
within rtol 1e-5 / atol 1e-5 of the float64 oracle), on calls in a row with shrinking
inputs - the array keeps the previous call's contents - and on inputs whose tiles need
the exact fix-up (the flags live in the array too)."""
import ctypes

import pytest
import torch

import oracle
from genbmm_amd import _lib

pytestmark = pytest.mark.gpu


def both(lib, gpu, a, b):
    B, M, K = a.shape
    N = b.shape[2]
    ad, bd = a.to(gpu), b.to(gpu)
    p, s = _lib.ptr, _lib.stream_of(ad)
    want = torch.full((B, M, N), float("nan"), device=gpu)
    stats = torch.empty(lib.genbmm_logbmm_stats_size(B, M, K, N), device=gpu)
    assert lib.genbmm_logbmm_fwd(p(ad), p(bd), p(want), p(stats), B, M, K, N, s) == 0
    got = torch.full((B, M, N), float("nan"), device=gpu)
    torch.cuda.synchronize()
    held = torch.cuda.memory_allocated()
    assert lib.genbmm_logbmm_fwd_static(p(ad), p(bd), p(got), B, M, K, N, s) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == held
    return got, want


def test_static_workspace_forward_matches_the_allocating_one(gpu):
    lib = _lib.load()
    torch.manual_seed(5)
    # matrix-core tiles (one batch item with rows that defeat the factoring -> flagged
    # tiles), then smaller: ragged matrix-core, one tile per item, vector-ALU tiles, whole-item kernels
    shapes = [(6, 256, 128, 256), (3, 130, 97, 200), (5, 128, 100, 96), (4, 70, 33, 50), (9, 32, 32, 32),
              (2, 5, 3, 4)]
    for rep in range(2):          # the second round starts from the smallest shape's leftovers
        for B, M, K, N in shapes:
            a, b = torch.randn(B, M, K), torch.randn(B, K, N)
            a[0, ::2, 0] += 200.0
            b[0, 0, :] -= 200.0
            got, want = both(lib, gpu, a, b)
            assert torch.equal(got, want), (rep, B, M, K, N)
            ref = torch.cat([oracle.logbmm_broadcast(a[i:i + 1].double(), b[i:i + 1].double()) for i in range(B)])
            assert torch.allclose(got.cpu().double(), ref, rtol=1e-5, atol=1e-5), (rep, B, M, K, N)


def test_static_workspace_limit(gpu):
    lib = _lib.load()
    limit = lib.genbmm_logbmm_static_limit()
    assert limit == 1 << 20
    t = torch.zeros(8, device=gpu)
    p, null = _lib.ptr, ctypes.c_void_p(0)
    B = limit // 64 + 1                      # B * (32 + 32) floats of maxima alone exceed the array
    assert lib.genbmm_logbmm_fwd_static(p(t), p(t), p(t), B, 32, 32, 32, null) == -5
    assert b"fixed workspace" in lib.genbmm_error_string(-5)
    assert lib.genbmm_logbmm_fwd_static(null, p(t), p(t), 1, 2, 2, 2, null) == -1
