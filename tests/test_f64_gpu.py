"""GPU parity of the double-precision entry points (`*_f64`) against the CPU oracle's
double instantiation of the reference kernels, through the public API and the C ABI."""
import numpy as np
import pytest
import torch

import oracle
import genbmm_amd as genbmm
from genbmm_amd import _lib
from genbmm_amd.sparse import BandedMatrix, banddiag

pytestmark = pytest.mark.gpu
F64 = np.float64
SHAPES = [(3, 9, 12, 7), (2, 33, 70, 129), (4, 64, 64, 64), (2, 1, 1, 1), (1, 130, 5, 66)]


def close(x, ref, rtol=1e-12, atol=1e-12):
    x, ref = x.detach().cpu(), ref.detach().cpu()
    assert x.dtype == torch.float64 and ref.dtype == torch.float64
    assert torch.allclose(x, ref, rtol=rtol, atol=atol), float((x - ref).abs().max())


def grid(*shape):
    return (torch.round(torch.randn(*shape) * 8) / 8).double()


@pytest.mark.parametrize("B,M,K,N", SHAPES)
def test_logbmm_f64(gpu, B, M, K, N):
    torch.manual_seed(K)
    a, b, g = torch.randn(B, M, K).double() * 3, torch.randn(B, K, N).double() * 3, torch.randn(B, M, N).double()
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = genbmm.logbmm(ad, bd)
    assert out.dtype == torch.float64
    close(out, oracle.seq_logbmm_fwd(a, b, dtype=F64)[0])
    close(out, oracle.logbmm_broadcast(a, b))
    ga, gb = torch.autograd.grad(out, (ad, bd), g.to(gpu), create_graph=True)
    wa, wb = oracle.seq_logbmm_bwd(a, b, g, dtype=F64)
    close(ga, wa)
    close(gb, wb)
    _, wa64, wb64 = oracle.logbmm_grads64(a, b, g)
    close(ga, wa64, 1e-10, 1e-12)
    close(gb, wb64, 1e-10, 1e-12)
    # second order: gradients of <u_a, grad_a> + <u_b, grad_b>
    ua, ub = torch.randn(B, M, K).double(), torch.randn(B, K, N).double()
    got = torch.autograd.grad((ga * ua.to(gpu)).sum() + (gb * ub.to(gpu)).sum(), (ad, bd))
    want = oracle.logbmm_second_order64(a, b, g, ua, ub)
    close(got[0], want[0], 1e-9, 1e-11)
    close(got[1], want[1], 1e-9, 1e-11)


@pytest.mark.parametrize("B,M,K,N", [(9, 128, 128, 128), (11, 100, 97, 120), (3, 200, 130, 96), (2, 65, 300, 129)])
def test_logbmm_f64_wide_tiles(gpu, B, M, K, N):
    """Shapes on the eight-wave 128 x 128 tiles: items that are one tile per gradient (both gradients
    in one launch), ragged edges, several tiles per item; one item needs the exact loops."""
    torch.manual_seed(B + N)
    a, b, g = torch.randn(B, M, K).double() * 3, torch.randn(B, K, N).double() * 3, torch.randn(B, M, N).double()
    a[1, ::3, 0] += 800.0
    b[1, 0, :] -= 800.0
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = genbmm.logbmm(ad, bd)
    close(out, oracle.logbmm_broadcast(a, b), 1e-12, 1e-9)
    ga, gb = torch.autograd.grad(out, (ad, bd), g.to(gpu))
    _, wa, wb = oracle.logbmm_grads64(a, b, g)
    close(ga, wa, 1e-10, 1e-9)
    close(gb, wb, 1e-10, 1e-9)
    close(ga.sum(-1), g.sum(-1), 1e-10, 1e-9)


def test_logbmm_f64_special_values(gpu):
    a = torch.tensor([[[0.0, -1e9, float("-inf")], [5.0, 5.0, 5.0]]], dtype=torch.float64)
    b = torch.zeros(1, 3, 2, dtype=torch.float64)
    out = genbmm.logbmm(a.to(gpu), b.to(gpu)).cpu()
    assert torch.allclose(out[0, 0], torch.zeros(2, dtype=torch.float64), atol=1e-15)
    assert torch.allclose(out[0, 1], torch.full((2,), 5 + np.log(3.0), dtype=torch.float64), rtol=1e-15)
    # a term float32 loses: log(1 + e^-30) = 9.36e-14, within the rounding of 1 + e^-30
    tiny = torch.tensor([[[0.0, -30.0]]], dtype=torch.float64)
    got = genbmm.logbmm(tiny.to(gpu), torch.zeros(1, 2, 1, dtype=torch.float64, device=gpu)).item()
    assert abs(got - np.log1p(np.exp(-30.0))) < 3e-16 and got != 0.0


def test_logbmm_f64_factoring_guard(gpu):
    """Shapes that take the factored matrix-core kernels, with rows and columns whose maxima
    sit on cells that never meet (exp(a - rowmax) * exp(b - colmax) underflows although the
    true terms do not), entries at the reference's -1e9 floor, -inf entries and a row that is
    all -inf: every such cell and every gradient fed by it must come from the exact loops."""
    torch.manual_seed(11)
    B, M, K, N = 2, 70, 40, 97
    a, b = torch.randn(B, M, K).double() * 3, torch.randn(B, K, N).double() * 3
    g = torch.randn(B, M, N).double()
    a[:, ::3, 0] += 800.0    # the row maximum, on k = 0 ...
    b[:, 0, :] -= 800.0      # ... which every column makes irrelevant
    b[:, 5, 1::4] += 700.0   # column maxima on k = 5
    a[0, 7, 3:9] = float("-inf")
    a[1, 10, :] = -1e9
    a[1, 20, :] = float("-inf")
    out = genbmm.logbmm(a.to(gpu), b.to(gpu)).cpu()
    want = oracle.seq_logbmm_fwd(a, b, dtype=F64)[0]
    live = torch.isfinite(want)
    assert bool(live.sum() > 0.9 * want.numel()) and torch.equal(torch.isfinite(out), live)
    close(out[live], want[live], 1e-12, 1e-9)
    close(out[live], oracle.logbmm_broadcast(a, b)[live], 1e-12, 1e-9)
    # gradients, without the all -inf row (its weights are NaN in the reference's own arithmetic)
    a[1, 20, :] = torch.randn(K).double()
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    ga, gb = torch.autograd.grad(genbmm.logbmm(ad, bd), (ad, bd), g.to(gpu))
    wa, wb = oracle.seq_logbmm_bwd(a, b, g, dtype=F64)
    assert torch.isfinite(wa).all() and torch.isfinite(wb).all()
    close(ga, wa, 1e-10, 1e-9)
    close(gb, wb, 1e-10, 1e-9)


# beside SHAPES: several slabs of 16 with a cut last one, reduction axes longer than one workgroup of
# the backward covers (128 cells of a column, 2048 of a row), tiles cut in both directions
MAX_SHAPES = SHAPES + [(2, 20, 300, 24), (1, 5, 2100, 3), (3, 70, 40, 130), (1, 64, 16, 64), (2, 67, 17, 4)]


@pytest.mark.parametrize("B,M,K,N", MAX_SHAPES)
@pytest.mark.parametrize("prod", [False, True])
def test_max_f64_bit_exact(gpu, B, M, K, N, prod):
    torch.manual_seed(M + N)
    if prod:
        a, b = (1 - torch.rand(B, M, K)).double(), (1 - torch.rand(B, K, N)).double()
        a[:, :, ::3] = torch.round(a[:, :, ::3] * 4) / 4 + 0.25
        b[:, ::3, :] = torch.round(b[:, ::3, :] * 4) / 4 + 0.25
        op = genbmm.prodmaxbmm
    else:
        a, b = grid(B, M, K), grid(B, K, N)
        op = genbmm.maxbmm
    g = grid(B, M, N).clamp(-4, 4)
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = op(ad, bd)
    sv, si = oracle.seq_maxbmm_fwd(a, b, prod, dtype=F64)
    assert out.dtype == torch.float64 and torch.equal(out.detach().cpu(), sv)
    ga, gb = torch.autograd.grad(out, (ad, bd), g.to(gpu))
    wa, wb = oracle.seq_argmax_bwd(a if prod else K, b, si, g, prod, dtype=F64)
    assert torch.equal(ga.cpu(), wa) and torch.equal(gb.cpu(), wb)
    # index through the C ABI
    lib = _lib.load()
    o2 = torch.empty(B, M, N, dtype=torch.float64, device=gpu)
    i2 = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
    fn = lib.genbmm_prodmaxbmm_fwd_f64 if prod else lib.genbmm_maxbmm_fwd_f64
    assert fn(_lib.ptr(ad.detach()), _lib.ptr(bd.detach()), _lib.ptr(o2), _lib.ptr(i2), B, M, K, N,
              _lib.stream_of(o2)) == 0
    assert torch.equal(i2.cpu(), si) and torch.equal(o2.cpu(), sv)


@pytest.mark.parametrize("B,M,K,N", [(2, 70, 261, 65), (1, 40, 600, 130), (3, 33, 7, 20), (2, 64, 512, 128)])
@pytest.mark.parametrize("prod", [False, True])
def test_max_f64_index_groups_and_special_values(gpu, prod, B, M, K, N):
    """The double-precision forward keeps the group of four consecutive k that last raised a
    cell's maximum and forms that group's terms again at the end: K across many slabs and not a
    multiple of the group, many ties, NaN / infinite / signed-zero terms, everything below the
    -1e9 floor.  Values are compared as bit patterns."""
    torch.manual_seed(K + N)
    a, b = grid(B, M, K) / 2, grid(B, K, N) / 2
    if prod:
        a, b = a.abs(), b.abs()       # zeros stay: products tie at 0 and signs of zero matter
        b[:, 1::5, :] *= -1
    a[:, ::7, 3::11] = float("nan")
    a[:, 1::9, 2::13] = float("inf")
    b[:, 4::17, ::6] = float("-inf")
    b[:, 5::19, 1::4] = -0.0
    a[:, 2::5, 5::19] = -0.0
    a[0, 0, :] = -0.0                 # a whole row of zero terms of both signs
    b[0, :, 0] = torch.where(torch.arange(K) % 3 == 0, 0.0, -0.0).double()
    if not prod:
        a[-1, 3, :] = -3e9            # every term of the row below the floor: value -1e9, index -1
    lib = _lib.load()
    ad, bd = a.to(gpu), b.to(gpu)
    out = torch.empty(B, M, N, dtype=torch.float64, device=gpu)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
    fn = lib.genbmm_prodmaxbmm_fwd_f64 if prod else lib.genbmm_maxbmm_fwd_f64
    assert fn(_lib.ptr(ad), _lib.ptr(bd), _lib.ptr(out), _lib.ptr(idx), B, M, K, N, _lib.stream_of(out)) == 0
    sv, si = oracle.seq_maxbmm_fwd(a, b, prod, dtype=F64)
    assert torch.equal(idx.cpu(), si)
    assert torch.equal(out.cpu().view(torch.int64), sv.view(torch.int64))
    assert int((si >= 0).sum()) > 0
    if not prod:
        assert bool((si[-1, 3] == -1).all()) and bool((sv[-1, 3] == -1e9).all())


def test_max_f64_at_the_benchmark_size(gpu):
    """(512,128,128,128) on the 1/8 grid (max) and Uniform(0,1] (prod-max), EVERY batch item: values
    and indices bit-exact against the broadcast closed form evaluated on the device in float64
    (index = the lowest k that attains the maximum); max gradients bit-exact against the one-hot
    scatter (g on the 1/8 grid: the sums are exact in any order), prod-max gradients against the
    scatter to rtol 1e-12; three items bit-exact against the sequential oracle, which also pins
    the order of the prod-max sums."""
    torch.manual_seed(1)
    B, M, K, N = 512, 128, 128, 128
    g = grid(B, M, N).clamp(-4, 4)
    gd = g.to(gpu)
    for prod in (False, True):
        if prod:
            a, b = (1 - torch.rand(B, M, K)).double(), (1 - torch.rand(B, K, N)).double()
            op = genbmm.prodmaxbmm
        else:
            a, b = grid(B, M, K), grid(B, K, N)
            op = genbmm.maxbmm
        ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
        out = op(ad, bd)
        ga, gb = torch.autograd.grad(out, (ad, bd), gd)
        lib = _lib.load()
        o2 = torch.empty(B, M, N, dtype=torch.float64, device=gpu)
        idx = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
        fn = lib.genbmm_prodmaxbmm_fwd_f64 if prod else lib.genbmm_maxbmm_fwd_f64
        assert fn(_lib.ptr(ad.detach()), _lib.ptr(bd.detach()), _lib.ptr(o2), _lib.ptr(idx), B, M, K, N,
                  _lib.stream_of(o2)) == 0
        pick = [0, 300, 511]
        sv, si = oracle.seq_maxbmm_fwd(a[pick], b[pick], prod, dtype=F64)
        assert torch.equal(out[pick].detach().cpu(), sv) and torch.equal(idx[pick].cpu(), si)
        wa, wb = oracle.seq_argmax_bwd(a[pick] if prod else K, b[pick], si, g[pick], prod, dtype=F64)
        assert torch.equal(ga[pick].cpu(), wa) and torch.equal(gb[pick].cpu(), wb)
        ks = torch.arange(K, device=gpu).view(1, 1, K, 1)
        ties = 0
        for i in range(0, B, 64):
            sl = slice(i, i + 64)
            x, y = ad[sl].detach().unsqueeze(-1), bd[sl].detach().unsqueeze(-3)
            s = x * y if prod else x + y                                          # (64, M, K, N)
            mv = s.max(-2).values
            hit = s == mv.unsqueeze(-2)
            first = torch.where(hit, ks, torch.full_like(ks, K)).min(-2).values
            assert torch.equal(out[sl].detach(), mv) and torch.equal(o2[sl], mv), i
            assert torch.equal(idx[sl].long(), first), i
            ties += int((hit.sum(-2) > 1).sum())
            wa64 = torch.zeros(64, M, K, device=gpu, dtype=torch.float64)
            wb64 = torch.zeros(64, K, N, device=gpu, dtype=torch.float64)
            if prod:
                bsel = torch.gather(bd[sl].detach(), 1, first)
                asel = torch.gather(ad[sl].detach().unsqueeze(2).expand(64, M, N, K), 3, first.unsqueeze(-1)).squeeze(-1)
                wa64.scatter_add_(2, first, bsel * gd[sl])
                wb64.scatter_add_(1, first, asel * gd[sl])
                assert torch.allclose(ga[sl], wa64, rtol=1e-12, atol=1e-12), i
                assert torch.allclose(gb[sl], wb64, rtol=1e-12, atol=1e-12), i
            else:
                wa64.scatter_add_(2, first, gd[sl])
                wb64.scatter_add_(1, first, gd[sl])
                assert torch.equal(ga[sl], wa64) and torch.equal(gb[sl], wb64), i
            del s, hit, first, mv
        if not prod:
            assert ties > 100 * B   # ties are present and resolve to the lowest k


def test_sample_f64_follows_the_cdf_rule(gpu):
    """Index = the reference's walk (matmul_cuda_kernel.cu:109-118) on the uniform of the
    cell, which is the float path's Philox draw for the same seed and offset."""
    torch.manual_seed(4)
    B, M, K, N = 3, 20, 37, 24
    a, b = torch.randn(B, M, K).double() * 2, torch.randn(B, K, N).double() * 2
    seed, offset = 1234, 8
    lib = _lib.load()
    ad, bd = a.to(gpu), b.to(gpu)
    out = torch.empty(B, M, N, dtype=torch.float64, device=gpu)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
    assert lib.genbmm_samplebmm_fwd_f64(_lib.ptr(ad), _lib.ptr(bd), _lib.ptr(out), _lib.ptr(idx), seed, offset,
                                        B, M, K, N, _lib.stream_of(ad)) == 0
    close(out, oracle.logbmm_broadcast(a, b))
    u = oracle.philox_uniform(0, B * M * N, seed, offset).view(B, M, N).double()
    sv, si = oracle.seq_samplebmm_fwd(a, b, u, dtype=F64)
    got = idx.cpu()
    # exp() of the device library and the host's differ in the last bits: a draw within
    # that distance of a CDF step may land on the neighbouring index
    assert float((got != si).float().mean()) < 1e-3
    cdf = oracle.sample_cdf64(a, b)
    gl = got.long()
    hi = torch.gather(cdf, 2, gl.unsqueeze(2)).squeeze(2)
    lo = torch.where(gl > 0, torch.gather(cdf, 2, (gl - 1).clamp(min=0).unsqueeze(2)).squeeze(2), torch.zeros_like(hi))
    assert bool(((lo - 1e-12 <= u) & (u <= hi + 1e-12)).all())
    # the float entry point draws the same uniforms: same index wherever float rounding allows
    o32 = torch.empty(B, M, N, device=gpu)
    i32 = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
    assert lib.genbmm_samplebmm_fwd(_lib.ptr(ad.float()), _lib.ptr(bd.float()), _lib.ptr(o32), _lib.ptr(i32),
                                    _lib.ptr(None), seed, offset, B, M, K, N, _lib.stream_of(ad)) == 0
    assert float((i32.cpu() != got).float().mean()) < 5e-3
    # through autograd: the gradient is the one-hot of the index times g
    ar, br = ad.clone().requires_grad_(True), bd.clone().requires_grad_(True)
    o = genbmm.samplebmm(ar, br, (seed, offset))
    g = torch.randn(B, M, N).double()
    ga, gb = torch.autograd.grad(o, (ar, br), g.to(gpu))
    onehot = torch.nn.functional.one_hot(got.long(), K).double()          # (B, M, N, K)
    assert torch.allclose(ga.cpu(), (onehot * g.unsqueeze(-1)).sum(2), rtol=1e-12, atol=1e-12)
    assert torch.allclose(gb.cpu().sum(1), g.sum(1), rtol=1e-12, atol=1e-12)


BANDS = [(5, 1, 1, 2, 0), (7, 0, 2, 2, 0), (3, 4, 5, 5, 4), (40, 3, 5, 4, 2), (130, 17, 2, 5, 20)]


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", BANDS)
@pytest.mark.parametrize("mode", [0, 1, 3])
def test_banded_f64(gpu, n, a_lu, a_ld, b_lu, b_ld, mode):
    torch.manual_seed(n + mode)
    exact = mode == 1
    mk = grid if exact else (lambda *s: torch.randn(*s).double())
    a = banddiag(mk(3, n, n), a_lu, a_ld)[0].contiguous()
    b = banddiag(mk(3, n, n), b_lu, b_ld)[0].contiguous()
    W = a.shape[2] + b.shape[2] - 1
    g = grid(3, n, W).clamp(-4, 4) if exact else torch.randn(3, n, W).double()
    X = BandedMatrix(a.to(gpu).requires_grad_(True), a_lu, a_ld)
    Y = BandedMatrix(b.to(gpu).requires_grad_(True), b_lu, b_ld)
    res = {0: X.multiply_log, 1: X.multiply_max, 3: X.multiply}[mode](Y)
    assert res.data.dtype == torch.float64
    want, widx, _ = oracle.seq_band_fwd(a, a_lu, a_ld, b, b_lu, b_ld, mode, dtype=F64)
    if exact:
        assert torch.equal(res.data.detach().cpu(), want)
    else:
        close(res.data, want, 1e-12, 1e-12)
    ga, gb = torch.autograd.grad(res.data, (X.data, Y.data), g.to(gpu), create_graph=(mode == 0))
    wa, wb = oracle.seq_band_bwd(a, a_lu, a_ld, b, b_lu, b_ld, g, mode, dtype=F64)
    if exact:
        assert torch.equal(ga.cpu(), wa) and torch.equal(gb.cpu(), wb)
    else:
        close(ga, wa, 1e-11, 1e-12)
        close(gb, wb, 1e-11, 1e-12)
    if mode == 0 and n <= 40:
        u = torch.randn_like(a)
        got = torch.autograd.grad((ga * u.to(gpu)).sum(), (X.data, Y.data))
        want = oracle.seq_band_bwdbwd(a, a_lu, a_ld, b, b_lu, b_ld, g, u, dtype=F64)
        close(got[0], want[0], 1e-10, 1e-11)
        close(got[1], want[1], 1e-10, 1e-11)


def test_f64_and_f32_disagree_only_by_float_rounding(gpu):
    torch.manual_seed(0)
    a, b = torch.randn(4, 64, 96), torch.randn(4, 96, 80)
    o32 = genbmm.logbmm(a.to(gpu), b.to(gpu)).double().cpu()
    o64 = genbmm.logbmm(a.double().to(gpu), b.double().to(gpu)).cpu()
    assert torch.allclose(o32, o64, rtol=1e-5, atol=1e-5) and not torch.equal(o32, o64)
    with pytest.raises(RuntimeError):
        genbmm.logbmm(a.double().to(gpu), b.to(gpu))
