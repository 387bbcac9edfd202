"""GPU parity of the banded sample product (`BandedMatrix.multiply_sample`,
genbmm_banded_sample_fwd) against the CPU oracle (all marked gpu).

The reference's band kernel has no sampling mode (banded_cuda_kernel.cu:42, 65, 76); the
rule is its dense one (matmul_cuda_kernel.cu:107-118) on a band cell's terms, restated in
oracle.seq_band_sample_fwd and pinned in tests/test_oracle.py.  Checked here: out against
the float64 log product; every index is a term of its cell and brackets the cell's Philox
uniform in the float64 CDF (tolerance 2e-5: the walk is fp32); fewer than 0.2 % of the
indices differ from the float64 rule; a chi-square bound on the draws; the one-hot
gradients bit for bit on dyadic data.
"""
import numpy as np
import pytest
import torch

import oracle
import genbmm_amd as genbmm
from genbmm_amd import _lib
from genbmm_amd.sparse import BandedMatrix, banddiag

pytestmark = pytest.mark.gpu

# narrow bands (one lane per cell), bands on the whole-strip walk (from 8 diagonals), matrix
# edges inside every strip, bands wider than the matrix, wide results cut into segments
BANDS = [(5, 1, 1, 2, 0), (7, 0, 2, 2, 0), (3, 4, 5, 5, 4), (33, 0, 0, 0, 0), (64, 8, 8, 8, 8), (130, 17, 2, 5, 20),
         (257, 32, 32, 32, 32), (200, 4, 4, 5, 5), (100, 60, 50, 40, 70), (300, 48, 48, 48, 48), (330, 120, 120, 120, 120)]


def pair(n, a_lu, a_ld, b_lu, b_ld, batch=3, scale=2.0):
    a = scale * banddiag(torch.randn(batch, n, n), a_lu, a_ld)[0].contiguous()
    b = scale * banddiag(torch.randn(batch, n, n), b_lu, b_ld)[0].contiguous()
    return a, b


def draw(gpu, a, a_lu, a_ld, b, b_lu, b_ld, seed, offset, use_ws=True):
    lib = _lib.load()
    B, n, Wa = a.shape
    Wo = Wa + b.shape[2] - 1
    out = torch.empty(B, n, Wo, device=gpu)
    idx = torch.empty(B, n, Wo, dtype=torch.int32, device=gpu)
    ws = None
    if use_ws:
        ws = torch.empty(lib.genbmm_banded_workspace_size(a_lu, a_ld, b_lu, b_ld, B, n), device=gpu)
    rc = lib.genbmm_banded_sample_fwd(_lib.ptr(a), a_lu, a_ld, _lib.ptr(b), b_lu, b_ld, _lib.ptr(out), _lib.ptr(idx),
                                      _lib.ptr(ws), seed, offset, B, n, _lib.stream_of(a))
    assert rc == 0
    return out, idx


def check_draw(a, a_lu, a_ld, b, b_lu, b_ld, out, idx, u, tol=2e-5):
    """a, b, out, idx, u on one device (the CDF is evaluated there in float64)."""
    cdf, valid = oracle.band_sample_cdf64(a, a_lu, a_ld, b, b_lu, b_ld)
    v, _ = oracle.band_terms64(a, a_lu, a_ld, b, b_lu, b_ld)
    inside = valid.any(-1)                                            # (n, Wo)
    want = v.logsumexp(-1)
    err = (out.double() - want).abs()[:, inside]
    assert float(err.max()) <= 1e-5 + 1e-5 * float(want[:, inside].abs().max()), float(err.max())
    assert bool((out[:, ~inside] == 0).all()) and bool((idx[:, ~inside] == 0).all())
    got = idx.long()
    assert int(got.min()) >= 0 and int(got.max()) < a.shape[2]
    is_term = torch.gather(valid.expand(a.shape[0], -1, -1, -1), 3, got.unsqueeze(-1)).squeeze(-1)
    assert bool(is_term[:, inside].all())
    hi = torch.gather(cdf, 3, got.unsqueeze(-1)).squeeze(-1)
    lo = torch.where(got > 0, torch.gather(cdf, 3, (got - 1).clamp(min=0).unsqueeze(-1)).squeeze(-1),
                     torch.zeros_like(hi))
    ud = u.double()
    ok = (lo - tol <= ud) & (ud <= hi + tol)
    assert bool(ok[:, inside].all()), float((~ok[:, inside]).float().mean())
    rule = oracle.band_sample_index_from_cdf(cdf, valid, ud).long()
    assert float((got != rule)[:, inside].float().mean()) < 2e-3


@pytest.mark.parametrize("use_ws", [True, False])
@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", BANDS)
def test_banded_sample_index_brackets_cdf(gpu, use_ws, n, a_lu, a_ld, b_lu, b_ld):
    torch.manual_seed(n + a_lu)
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld)
    ad, bd = a.to(gpu), b.to(gpu)
    seed, offset = 1234, 9
    out, idx = draw(gpu, ad, a_lu, a_ld, bd, b_lu, b_ld, seed, offset, use_ws)
    u = oracle.philox_uniform(0, out.numel(), seed, offset).view(out.shape)
    check_draw(a, a_lu, a_ld, b, b_lu, b_ld, out.cpu(), idx.cpu(), u)
    # the sequential fp32 restatement on the same uniforms agrees almost everywhere
    _, sidx = oracle.seq_band_sample_fwd(a, a_lu, a_ld, b, b_lu, b_ld, u)
    assert float((idx.cpu() != sidx).float().mean()) < 2e-3
    # same stream -> same draw; another offset -> another draw (where there is a choice)
    _, idx2 = draw(gpu, ad, a_lu, a_ld, bd, b_lu, b_ld, seed, offset, use_ws)
    assert torch.equal(idx, idx2)
    _, idx3 = draw(gpu, ad, a_lu, a_ld, bd, b_lu, b_ld, seed, offset + 1, use_ws)
    if a.shape[2] > 1 and b.shape[2] > 1:
        assert not torch.equal(idx, idx3)


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", [(70, 3, 5, 4, 2), (200, 20, 12, 9, 30), (64, 8, 8, 8, 8)])
def test_banded_sample_cells_that_need_the_exact_walk(gpu, n, a_lu, a_ld, b_lu, b_ld):
    """Band rows whose maxima sit on cells that never meet (the factored sums underflow), -inf
    entries and a fully masked row: those cells have no usable 1/S and walk exactly."""
    torch.manual_seed(n)
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld, scale=1.0)
    a[:, ::3, 0] += 150.0
    b[:, :, 0] -= 150.0
    b[:, 1::4, -1] += 120.0
    a[1, 5:9, 1:3] = -float("inf")
    out, idx = draw(gpu, a.to(gpu), a_lu, a_ld, b.to(gpu), b_lu, b_ld, 77, 0)
    u = oracle.philox_uniform(0, out.numel(), 77, 0).view(out.shape)
    check_draw(a, a_lu, a_ld, b, b_lu, b_ld, out.cpu(), idx.cpu(), u)


def test_banded_sample_chi_square(gpu):
    """2 x 10^4 draws (batch items of the same small band pair, one Philox stream) per cell
    against the float64 softmax of the cell's terms; categories with expected count < 5
    pooled; bound = the 1 - 1e-6 quantile."""
    from scipy.stats import chi2 as chi2_dist

    torch.manual_seed(3)
    n, a_lu, a_ld, b_lu, b_ld, draws = 24, 5, 6, 4, 7, 20000
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld, batch=1)
    for use_ws in (True, False):
        A, Bm = a.expand(draws, -1, -1).contiguous().to(gpu), b.expand(draws, -1, -1).contiguous().to(gpu)
        _, idx = draw(gpu, A, a_lu, a_ld, Bm, b_lu, b_ld, 5, 11, use_ws)
        cdf, valid = oracle.band_sample_cdf64(a, a_lu, a_ld, b, b_lu, b_ld)
        pr = torch.diff(cdf[0], dim=-1, prepend=torch.zeros(n, cdf.shape[2], 1, dtype=torch.float64))
        Wa, Wo = a.shape[2], idx.shape[2]
        counts = torch.zeros(n * Wo, Wa, device=gpu)
        cells = torch.arange(n * Wo, device=gpu).repeat(draws)
        counts.index_put_((cells, idx.reshape(-1).long()), torch.ones(draws * n * Wo, device=gpu), accumulate=True)
        counts = counts.cpu().double().view(n, Wo, Wa)
        for i in range(n):
            for j in range(Wo):
                if not valid[i, j].any():
                    continue
                e, c = pr[i, j] * draws, counts[i, j]
                keep = e >= 5
                stat, dof = float((((c - e) ** 2) / e)[keep].sum()), int(keep.sum())
                if (~keep).any() and float(e[~keep].sum()) >= 1:
                    stat += (float(c[~keep].sum()) - float(e[~keep].sum())) ** 2 / float(e[~keep].sum())
                    dof += 1
                assert stat < chi2_dist.ppf(1 - 1e-6, max(dof - 1, 1)), (use_ws, i, j, stat, dof)


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", [(40, 3, 5, 4, 2), (257, 32, 32, 32, 32), (100, 60, 50, 40, 70)])
def test_banded_sample_gradients_are_the_one_hot_scatter(gpu, n, a_lu, a_ld, b_lu, b_ld):
    torch.manual_seed(n)
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld)
    B, _, Wa = a.shape
    Wb = b.shape[2]
    Wo = Wa + Wb - 1
    g = (torch.round(torch.randn(B, n, Wo) * 8) / 8).clamp(-4, 4)    # dyadic: sums are exact in any order
    X = BandedMatrix(a.to(gpu).requires_grad_(True), a_lu, a_ld)
    Y = BandedMatrix(b.to(gpu).requires_grad_(True), b_lu, b_ld)
    res = X.multiply_sample(Y, (42, 3))
    assert (res.lu, res.ld) == (a_lu + b_ld, a_ld + b_lu)
    ga, gb = torch.autograd.grad(res.data, (X.data, Y.data), g.to(gpu))
    out, idx = draw(gpu, X.data.detach(), a_lu, a_ld, Y.data.detach(), b_lu, b_ld, 42, 3)
    assert torch.equal(out, res.data.detach())
    # grad_a[i, k] += g[i, j], grad_b[o, k2] += g[i, j] for k = idx[i, j], o = i + j - lu_out, k2 = k - j + Wb - 1
    idx = idx.cpu().long()
    i = torch.arange(n).view(1, n, 1).expand(B, n, Wo)
    j = torch.arange(Wo).view(1, 1, Wo).expand(B, n, Wo)
    o = i + j - (a_lu + b_ld)
    inside = (o >= 0) & (o < n)
    bb = torch.arange(B).view(B, 1, 1).expand(B, n, Wo)
    wa, wb = torch.zeros(B, n, Wa), torch.zeros(B, n, Wb)
    wa.index_put_((bb[inside], i[inside], idx[inside]), g[inside], accumulate=True)
    wb.index_put_((bb[inside], o[inside], (idx - j + Wb - 1)[inside]), g[inside], accumulate=True)
    assert torch.equal(ga.cpu(), wa) and torch.equal(gb.cpu(), wb)


def test_banded_sample_follows_torch_seed_and_double(gpu):
    a, b = pair(50, 6, 5, 4, 7)
    X = BandedMatrix(a.to(gpu).requires_grad_(True), 6, 5)
    Y = BandedMatrix(b.to(gpu), 4, 7)
    torch.manual_seed(5)
    g1 = torch.autograd.grad(X.multiply_sample(Y).data.sum(), X.data)[0]
    g2 = torch.autograd.grad(X.multiply_sample(Y).data.sum(), X.data)[0]
    torch.manual_seed(5)
    g3 = torch.autograd.grad(X.multiply_sample(Y).data.sum(), X.data)[0]
    assert torch.equal(g1, g3) and not torch.equal(g1, g2)
    # double precision: the same uniforms, the exact walk, equal to the sequential oracle
    Xd = BandedMatrix(a.double().to(gpu).requires_grad_(True), 6, 5)
    Yd = BandedMatrix(b.double().to(gpu).requires_grad_(True), 4, 7)
    res = Xd.multiply_sample(Yd, (9, 2))
    u = oracle.philox_uniform(0, res.data.numel(), 9, 2).view(res.data.shape).double()
    want, widx = oracle.seq_band_sample_fwd(a.double(), 6, 5, b.double(), 4, 7, u, dtype=np.float64)
    assert torch.allclose(res.data.detach().cpu(), want, rtol=1e-12, atol=1e-12)
    ga, gb = torch.autograd.grad(res.data.sum(), (Xd.data, Yd.data))
    hist = torch.zeros_like(a, dtype=torch.float64)
    inside = oracle.band_terms64(a, 6, 5, b, 4, 7)[1].any(-1)
    hist.scatter_add_(2, widx.long(), inside.expand_as(widx).double())
    assert float((ga.cpu() - hist).abs().sum()) <= 2e-3 * float(hist.sum())  # exp/log rounding at CDF steps


def test_banded_sample_config_c5_at_full_size(gpu):
    """The banded benchmark configuration (batch 64, n = 4096, 65 diagonals per operand, seed 7):
    out and indices of three batch items against the float64 CDF evaluated on the device,
    term validity and the gradient-sum invariant over everything."""
    torch.manual_seed(7)
    B, n, lu = 64, 4096, 32
    a, b = torch.rand(B, n, 2 * lu + 1) * 2 - 1, torch.rand(B, n, 2 * lu + 1) * 2 - 1
    ad, bd = a.to(gpu), b.to(gpu)
    out, idx = draw(gpu, ad, lu, lu, bd, lu, lu, 1234, 0)
    Wo = out.shape[2]
    for item in (0, 29, 63):
        u = oracle.philox_uniform(item * n * Wo, n * Wo, 1234, 0).view(1, n, Wo).to(gpu)
        for r0 in range(0, n, 1024):                                  # 1024 rows at a time, with their halo of b
            lo, hi = max(r0 - 2 * lu, 0), min(r0 + 1024 + 2 * lu, n)
            sub_a, sub_b = ad[item:item + 1, lo:hi], bd[item:item + 1, lo:hi]
            cdf, valid = oracle.band_sample_cdf64(sub_a, lu, lu, sub_b, lu, lu)
            rows = slice(r0 - lo, r0 - lo + 1024)
            # rows next to the cut see the sub-matrix's edge, not the matrix's: compare interior rows only
            keep = torch.zeros(hi - lo, dtype=torch.bool, device=gpu)
            keep[rows] = True
            if lo > 0:
                keep[: 2 * lu] = False
            if hi < n:
                keep[-2 * lu:] = False
            got = idx[item:item + 1, lo:hi].long()
            ui = u[:, lo:hi].double()
            hi_c = torch.gather(cdf, 3, got.unsqueeze(-1)).squeeze(-1)
            lo_c = torch.where(got > 0, torch.gather(cdf, 3, (got - 1).clamp(min=0).unsqueeze(-1)).squeeze(-1),
                               torch.zeros_like(hi_c))
            ok = ((lo_c - 2e-5 <= ui) & (ui <= hi_c + 2e-5)) | ~valid.any(-1)
            assert bool(ok[:, keep].all()), (item, r0)
            del cdf, valid
    g = (torch.round(torch.randn(B, n, Wo) * 8) / 8).clamp(-4, 4).to(gpu)
    ga, gb = torch.empty_like(ad), torch.empty_like(bd)
    lib = _lib.load()
    rc = lib.genbmm_banded_bwd(_lib.ptr(ad), lu, lu, _lib.ptr(bd), lu, lu, _lib.ptr(None), _lib.ptr(idx), _lib.ptr(None),
                               _lib.ptr(g), _lib.ptr(ga), _lib.ptr(gb), B, n, 2, _lib.stream_of(ad))
    assert rc == 0
    i = torch.arange(n, device=gpu).view(n, 1)
    o = i + torch.arange(Wo, device=gpu).view(1, Wo) - 2 * lu
    inside = (o >= 0) & (o < n)
    assert torch.equal(ga.sum(-1), (g * inside).sum(-1))
