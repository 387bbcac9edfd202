"""Many small and odd shapes through the arg-max products and their backward: the group
sweep + resolve (64- and 32-column panels, ragged K), the (line, k-range) backward with
one to sixty-four ranges, and samplebmm's three sweeps.  Seeded, so the cases are fixed."""
import random

import numpy as np
import pytest
import torch

import oracle
import genbmm_amd as genbmm
from genbmm_amd import _lib

pytestmark = pytest.mark.gpu


def _shapes(seed, count, kmax):
    rng = random.Random(seed)
    edge = [1, 2, 3, 7, 8, 9, 31, 32, 33, 63, 64, 65, 96, 97, 127, 128, 129, 130]
    out = []
    for _ in range(count):
        M = rng.choice(edge + [rng.randint(1, 200)])
        N = rng.choice(edge + [rng.randint(1, 200)])
        K = rng.choice([1, 2, 7, 8, 9, 15, 16, 17, 127, 128, 129, 255, 256, 257, 263, 511, 512, 513, rng.randint(1, kmax)])
        B = rng.randint(1, 3)
        if B * M * K * N > 6_000_000:
            K = max(1, 6_000_000 // (B * M * N))
        out.append((B, M, K, N))
    return out


def grid(*shape):
    return torch.round(torch.randn(*shape) * 4) / 4


@pytest.mark.parametrize("prod", [False, True])
def test_max_products_on_many_shapes(gpu, prod):
    torch.manual_seed(5)
    for B, M, K, N in _shapes(11 + prod, 40, 700):
        a, b = grid(B, M, K), grid(B, K, N)
        g = grid(B, M, N).clamp(-4, 4)
        ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
        out = (genbmm.prodmaxbmm if prod else genbmm.maxbmm)(ad, bd)
        sv, si = oracle.seq_maxbmm_fwd(a, b, prod)
        assert torch.equal(out.detach().cpu(), sv), (B, M, K, N)
        ga, gb = torch.autograd.grad(out, (ad, bd), g.to(gpu))
        wa, wb = oracle.seq_argmax_bwd(a if prod else K, b, si, g, prod)
        assert torch.equal(ga.cpu(), wa) and torch.equal(gb.cpu(), wb), (B, M, K, N)


def test_argmax_backward_with_many_k_ranges(gpu):
    """K from one range of 128 cells to more than 64 of them (several workgroups per line)."""
    lib = _lib.load()
    torch.manual_seed(6)
    for B, M, K, N in [(1, 5, 1, 9), (2, 70, 129, 33), (1, 40, 1000, 70), (1, 9, 4097, 17), (1, 3, 8200, 5),
                       (1, 2, 9000, 130)]:
        idx = torch.randint(-1, K, (B, M, N), dtype=torch.int32)
        g = torch.randn(B, M, N)
        ga = torch.full((B, M, K), float("nan"), device=gpu)
        gb = torch.full((B, K, N), float("nan"), device=gpu)
        assert lib.genbmm_argmax_bwd(_lib.ptr(idx.to(gpu)), _lib.ptr(g.to(gpu)), _lib.ptr(ga), _lib.ptr(gb),
                                     B, M, K, N, _lib.stream_of(ga)) == 0
        wa, wb = oracle.seq_argmax_bwd(K, torch.zeros(B, K, N), idx, g, False)
        assert torch.equal(ga.cpu(), wa) and torch.equal(gb.cpu(), wb), (B, M, K, N)


def test_sample_on_many_shapes(gpu):
    """Every index brackets its uniform in the float64 CDF; shapes on both sides of the
    matrix-core limits (M, N >= 96, K >= 16), of the 62 slabs that its six-bit tag counts
    (K <= 992; K = 993, 1008, 1040: seven bits) and of its 126-slab limit (K <= 2016; the last
    shape has a matrix-core forward and, with K = 2020, the two-level sweep on the vector ALU
    behind it)."""
    lib = _lib.load()
    torch.manual_seed(7)
    shapes = _shapes(13, 14, 400) + [(1, 96, 16, 96), (1, 97, 993, 100), (1, 130, 992, 96), (2, 100, 500, 131),
                                     (1, 128, 1040, 160), (2, 256, 1008, 128), (1, 128, 2016, 96), (1, 96, 2020, 128)]
    for B, M, K, N in shapes:
        a, b = 2 * torch.randn(B, M, K), 2 * torch.randn(B, K, N)
        ad, bd = a.to(gpu), b.to(gpu)
        out = torch.empty(B, M, N, device=gpu)
        idx = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
        stats = torch.empty(lib.genbmm_samplebmm_stats_size(B, M, K, N), device=gpu)
        assert lib.genbmm_samplebmm_fwd(_lib.ptr(ad), _lib.ptr(bd), _lib.ptr(out), _lib.ptr(idx), _lib.ptr(stats),
                                        77, 3, B, M, K, N, _lib.stream_of(ad)) == 0
        u = oracle.philox_uniform(0, B * M * N, 77, 3).view(B, M, N).double()
        cdf = oracle.sample_cdf64(a, b)
        got = idx.cpu().long()
        assert int(got.min()) >= 0 and int(got.max()) < K, (B, M, K, N)
        hi = torch.gather(cdf, 2, got.unsqueeze(2)).squeeze(2)
        lo = torch.where(got > 0, torch.gather(cdf, 2, (got - 1).clamp(min=0).unsqueeze(2)).squeeze(2),
                         torch.zeros_like(hi))
        ok = (lo - 2e-5 <= u) & (u <= hi + 2e-5)
        assert bool(ok.all()), ((B, M, K, N), float((~ok).float().mean()))
        want = oracle.sample_index_from_cdf(cdf, u).long()
        assert float((got != want).float().mean()) < 5e-3, (B, M, K, N)


@pytest.mark.parametrize("shape", [(2, 128, 200, 160), (2, 256, 512, 128)])
@pytest.mark.parametrize("scale", [0.05, 2.0, 12.0, 40.0, 100.0, 400.0])
def test_sample_on_flat_and_peaked_distributions(gpu, scale, shape):
    """From nearly uniform to one-term-takes-all (at the largest scales the winning term leads by
    hundreds: the remainder the matrix-core sweep hands to the resolve step, six mantissa bits
    short, must still name the right term), with masked terms (-inf, -1e9), on shapes that take
    the matrix-core sweep (and its exact fix-up where S underflows): 13 and 32 slabs."""
    lib = _lib.load()
    torch.manual_seed(int(scale * 10))
    B, M, K, N = shape
    a, b = scale * torch.randn(B, M, K), scale * torch.randn(B, K, N)
    a[:, ::3, ::5] = float("-inf")
    b[:, 1::7, ::2] = -1e9
    a[1, 5, :] = float("-inf")          # a row without any mass: out = -inf, index 0
    ad, bd = a.to(gpu), b.to(gpu)
    out = torch.empty(B, M, N, device=gpu)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
    stats = torch.empty(lib.genbmm_samplebmm_stats_size(B, M, K, N), device=gpu)
    assert lib.genbmm_samplebmm_fwd(_lib.ptr(ad), _lib.ptr(bd), _lib.ptr(out), _lib.ptr(idx), _lib.ptr(stats),
                                    5, 11, B, M, K, N, _lib.stream_of(ad)) == 0
    u = oracle.philox_uniform(0, B * M * N, 5, 11).view(B, M, N).double()
    want_out, want_idx = oracle.seq_samplebmm_fwd(a, b, u.float())
    got = idx.cpu().long()
    live = torch.ones(B, M, N, dtype=torch.bool)
    live[1, 5, :] = False
    assert bool((got[~live] == 0).all()) and bool((out.cpu()[~live] == want_out[~live]).all())
    assert torch.allclose(out.cpu()[live], want_out[live], rtol=1e-5, atol=1e-5)
    cdf = oracle.sample_cdf64(a, b)
    hi = torch.gather(cdf, 2, got.unsqueeze(2)).squeeze(2)
    lo = torch.where(got > 0, torch.gather(cdf, 2, (got - 1).clamp(min=0).unsqueeze(2)).squeeze(2), torch.zeros_like(hi))
    # fp32 prefix sums over K terms (the reference's too): K roundings of 2^-24 of the running mass;
    # and the masses are exp(a + b - out) with `out` rounded to fp32: 2^-24 |out| in the exponent
    tol = max(2e-5, 2.0 * K * 2.0 ** -24, 2.0 * float(want_out[live].abs().max()) * 2.0 ** -23)
    viol = torch.maximum(lo - u, u - hi).clamp(min=0)
    ok = (viol <= tol) | ~live
    assert bool(ok.all()), (float((~ok).float().mean()), float(viol[live].max()), tol)
    # a sampled term always has mass (never a masked one)
    picked = torch.gather(a.unsqueeze(-1) + b.unsqueeze(-3), 2, got.unsqueeze(2)).squeeze(2)
    assert bool((picked[live] > -1e8).all())
