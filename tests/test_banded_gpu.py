"""GPU parity of the banded products against the CPU oracle (all marked gpu)."""
import numpy as np
import pytest
import torch

import oracle
import genbmm_amd as genbmm
from genbmm_amd import _lib
from genbmm_amd.sparse import BandedMatrix, banddiag

pytestmark = pytest.mark.gpu

# (n, a_lu, a_ld, b_lu, b_ld): bands narrower and wider than the matrix, empty sides
BANDS = [(5, 1, 1, 2, 0), (6, 2, 1, 1, 3), (4, 3, 3, 3, 3), (7, 0, 2, 2, 0), (3, 4, 5, 5, 4),
         (40, 3, 5, 4, 2), (33, 0, 0, 0, 0), (64, 8, 8, 8, 8), (1, 0, 0, 0, 0), (130, 17, 2, 5, 20),
         (257, 32, 32, 32, 32), (100, 60, 50, 40, 70),
         # wide bands on the memory-fed matrix-core kernels (97 ... 201 diagonals, and a wide band
         # against a narrow one), and one beyond what they take (241 diagonals)
         (300, 48, 48, 48, 48), (260, 52, 49, 50, 50), (230, 64, 64, 64, 64), (420, 100, 100, 100, 100),
         (300, 120, 3, 2, 90), (330, 120, 120, 120, 120)]


def close(x, ref, rtol=1e-5, atol=1e-5):
    x, ref = x.detach().cpu().double(), ref.detach().cpu().double()
    assert torch.allclose(x, ref, rtol=rtol, atol=atol), float((x - ref).abs().max())


def grid(*shape):
    return torch.round(torch.randn(*shape) * 8) / 8


def pair(n, a_lu, a_ld, b_lu, b_ld, batch=3, mk=torch.randn):
    a = banddiag(mk(batch, n, n), a_lu, a_ld)[0].contiguous()
    b = banddiag(mk(batch, n, n), b_lu, b_ld)[0].contiguous()
    return a, b


@pytest.mark.parametrize("batch,n,a_lu,a_ld,b_lu,b_ld", [(2, 330, 120, 120, 120, 120), (2, 300, 150, 100, 90, 140),
                                                         (1, 260, 129, 129, 129, 129), (3, 700, 120, 120, 120, 120),
                                                         (2, 1400, 120, 120, 120, 120)])
@pytest.mark.parametrize("mode", [0, 3])
def test_very_wide_bands_multiply_as_dense_matrices(gpu, batch, n, a_lu, a_ld, b_lu, b_ld, mode):
    """Bands beyond what the matrix-core band kernels take (about 225 diagonals per operand): where
    the matrices are small enough, BandedMatrix.multiply / multiply_log go through to_dense, the
    dense product and banddiag instead of one lane per result cell.  Same values and gradients as the
    sequential oracle, cells of the bands outside the matrix holding anything; the last shape's log
    product (a band that leaves most of the dense result empty) stays on the band kernels, as do
    calls through the C ABI (the two routes agree)."""
    lib = _lib.load()
    assert lib.genbmm_banded_on_matrix_cores(a_lu, a_ld, b_lu, b_ld, batch, n) == 0
    assert lib.genbmm_banded_on_matrix_cores(32, 32, 32, 32, 64, 4096) == 1
    torch.manual_seed(n + mode)
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld, batch=batch)
    a[:, :3, :] += 100.0 * (a[:, :3, :] == 0)
    b[:, -3:, :] += 100.0 * (b[:, -3:, :] == 0)
    X = BandedMatrix(a.to(gpu).requires_grad_(True), a_lu, a_ld)
    Y = BandedMatrix(b.to(gpu).requires_grad_(True), b_lu, b_ld)
    assert X._dense_pays(Y, mode == 0) == (not (mode == 0 and n == 1400))
    res = (X.multiply_log if mode == 0 else X.multiply)(Y)
    assert (res.lu, res.ld) == (a_lu + b_ld, a_ld + b_lu)
    want, _, _ = oracle.seq_band_fwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, mode, dtype=np.float64)
    W = a.shape[2] + b.shape[2] - 1
    atol = 1e-5 * max(1.0, W / 64.0)
    close(res.data, want, atol=atol)
    g = torch.randn(batch, n, W)
    ga, gb = torch.autograd.grad(res.data, (X.data, Y.data), g.to(gpu))
    wa, wb = oracle.seq_band_bwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, g.double(), mode, dtype=np.float64)
    close(ga, wa, atol=atol)
    close(gb, wb, atol=atol)
    # the band kernels on the same operands (the autograd Functions called directly)
    fn = genbmm.sparse.bandedlogbmm if mode == 0 else genbmm.sparse.bandedbmm
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    direct = fn(ad, a_lu, a_ld, bd, b_lu, b_ld, a_lu + b_ld, a_ld + b_lu)
    close(direct, res.data, atol=atol)
    close(direct, want, atol=atol)
    da, db = torch.autograd.grad(direct, (ad, bd), g.to(gpu))
    close(da, wa, atol=atol)
    close(db, wb, atol=atol)


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", BANDS)
@pytest.mark.parametrize("mode", [0, 1, 3])
def test_banded_forward_backward(gpu, n, a_lu, a_ld, b_lu, b_ld, mode):
    torch.manual_seed(n * 7 + mode)
    exact = mode == 1
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld, mk=grid if exact else torch.randn)
    W = a.shape[2] + b.shape[2] - 1
    g = grid(3, n, W).clamp(-4, 4) if exact else torch.randn(3, n, W)
    X = BandedMatrix(a.to(gpu).requires_grad_(True), a_lu, a_ld)
    Y = BandedMatrix(b.to(gpu).requires_grad_(True), b_lu, b_ld)
    res = {0: X.multiply_log, 1: X.multiply_max, 3: X.multiply}[mode](Y)
    assert (res.lu, res.ld) == (a_lu + b_ld, a_ld + b_lu)
    # float64 sequential restatement of the reference kernel; whole tensor incl. zero cells
    want, widx, _ = oracle.seq_band_fwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, mode, dtype=np.float64)
    # fp32 sums of up to `terms` products of unit-variance values (their partial sums reach
    # sqrt(terms) times a few): the absolute error of a sum grows with its length, whatever the
    # size of the result (which may cancel to nothing); 1e-5 up to about 64 terms, as stated
    terms = max(a.shape[2], b.shape[2], W)
    atol = 1e-5 * max(1.0, terms / 64.0)
    if exact:
        assert torch.equal(res.data.detach().cpu().double(), want)
    else:
        close(res.data, want, atol=atol)
    ga, gb = torch.autograd.grad(res.data, (X.data, Y.data), g.to(gpu))
    wa, wb = oracle.seq_band_bwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, g.double(), mode, dtype=np.float64)
    if exact:
        assert torch.equal(ga.cpu().double(), wa) and torch.equal(gb.cpu().double(), wb)
    else:
        close(ga, wa, atol=atol)
        close(gb, wb, atol=atol)


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", [(70, 3, 5, 4, 2), (200, 20, 12, 9, 30), (64, 8, 8, 8, 8)])
def test_banded_log_factoring_guard(gpu, n, a_lu, a_ld, b_lu, b_ld):
    """Band rows whose maxima sit on cells that never meet: exp(a - rowmax) * exp(b - rowmax)
    underflows although the true terms do not; those cells / gradient rows must be recomputed
    exactly.  Also -inf entries (masked cells) and a fully masked row."""
    torch.manual_seed(n)
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld)
    a[:, ::3, 0] += 150.0            # first band cell of every third column of a
    b[:, :, 0] -= 150.0
    b[:, 1::4, -1] += 120.0
    a[1, 5:9, 1:3] = -float("inf")   # masked cells
    W = a.shape[2] + b.shape[2] - 1
    g = torch.randn(3, n, W)
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    res = BandedMatrix(ad, a_lu, a_ld).multiply_log(BandedMatrix(bd, b_lu, b_ld))
    want, _, _ = oracle.seq_band_fwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, 0, dtype=np.float64)
    close(res.data, want)
    ga, gb = torch.autograd.grad(res.data, (ad, bd), g.to(gpu))
    wa, wb = oracle.seq_band_bwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, g.double(), 0, dtype=np.float64)
    # a weight exp(a + b - out) evaluated in fp32 is as accurate as its argument: a, b and out
    # each carry half an ulp of their magnitude, and that absolute error of the argument is the
    # relative error of the weight
    scale = max(float(a[torch.isfinite(a)].abs().max()), float(b.abs().max()))
    tol = 4 * float(torch.finfo(torch.float32).eps) * scale
    assert 1e-5 < tol < 2e-4
    close(ga, wa, rtol=tol, atol=tol)
    close(gb, wb, rtol=tol, atol=tol)


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", [(200, 6, 5, 4, 7), (600, 32, 32, 32, 32), (300, 12, 20, 30, 3)])
def test_banded_log_rows_padded_at_the_floor(gpu, n, a_lu, a_ld, b_lu, b_ld):
    """Band rows written as -1e9 throughout (padding at the reference's floor,
    banded_cuda_kernel.cu:31-33): max_k(a + b) of their cells is -1e9 + max b, not below the
    floor, so the result is the plain log-sum-exp (float64: -1e9 + logsumexp of the cells of b
    it meets; a float near -1e9 is a multiple of 64).  No gradient flows into the padding;
    everything else must not notice it.  These rows are factored like any other (their 1 / S
    comes from the sums); where a padded row of a meets a padded row of b every term is at
    -2e9 and the per-cell routine gives the reference's -inf."""
    torch.manual_seed(n + a_lu)
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld)
    W = a.shape[2] + b.shape[2] - 1
    g = torch.randn(3, n, W)
    pad = slice(n - n // 6, n)
    a[:2, pad, :] = -1e9                      # the last rows of a (items 0, 1)
    b[1:, pad, :] = -1e9                      # the last rows of b (items 1, 2): item 1 has both
    want, _, _ = oracle.seq_band_fwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, 0, dtype=np.float64)
    want32, _, _ = oracle.seq_band_fwd(a, a_lu, a_ld, b, b_lu, b_ld, 0)
    at_floor = want < -5e8                    # cells fed by padding: near -1e9, or -inf in float where both meet
    g[at_floor] = 0.0
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    res = BandedMatrix(ad, a_lu, a_ld).multiply_log(BandedMatrix(bd, b_lu, b_ld))
    got = res.data.detach().cpu()
    gone = torch.isinf(want32)                # the reference's own float arithmetic: terms at -2e9 vanish
    assert torch.equal(torch.isinf(got), gone)
    close(got[~at_floor], want[~at_floor])
    close(got[at_floor & ~gone], want[at_floor & ~gone], rtol=0, atol=128.0)
    ga, gb = torch.autograd.grad(res.data, (ad, bd), g.to(gpu))
    wa, wb = oracle.seq_band_bwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, g.double(), 0, dtype=np.float64)
    # item 1, where results are -inf, has 0 * inf among its weights in the reference's own arithmetic
    ok = torch.tensor([0, 2])
    assert bool(torch.isfinite(ga[ok.to(gpu)]).all()) and bool(torch.isfinite(gb[ok.to(gpu)]).all())
    close(ga[ok.to(gpu)], wa[ok], atol=2e-5)
    close(gb[ok.to(gpu)], wb[ok], atol=2e-5)


def test_banded_max_index_through_c_abi(gpu):
    torch.manual_seed(2)
    n, a_lu, a_ld, b_lu, b_ld = 50, 4, 6, 5, 3
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld, mk=grid)
    ad, bd = a.to(gpu), b.to(gpu)
    W = a.shape[2] + b.shape[2] - 1
    out = torch.empty(3, n, W, device=gpu)
    idx = torch.empty(3, n, W, dtype=torch.int32, device=gpu)
    rc = _lib.load().genbmm_banded_fwd(_lib.ptr(ad), a_lu, a_ld, _lib.ptr(bd), b_lu, b_ld, _lib.ptr(out),
                                       _lib.ptr(idx), _lib.ptr(None), 3, n, 1, _lib.stream_of(ad))
    assert rc == 0
    want, widx, _ = oracle.seq_band_fwd(a, a_lu, a_ld, b, b_lu, b_ld, 1)
    assert torch.equal(out.cpu(), want) and torch.equal(idx.cpu(), widx)


@pytest.mark.parametrize("n,lu,ld", [(5, 3, 4), (4, 5, 3), (3, 3, 3), (9, 2, 4)])
def test_reference_style_log_product(gpu, n, lu, ld):
    """The reference's own banded test (test_cuda.py:46-49, 81-143):
    bmm(a, b) = b.multiply_log(a.transpose()), forward, gradients and second-order terms."""
    torch.manual_seed(n + lu)
    band, _ = banddiag(torch.rand(3, n, n), lu, ld)
    band2, _ = banddiag(torch.rand(3, n, n), lu, ld)
    back = torch.rand(3, n, 2 * (lu + ld) + 1)
    back2 = (torch.rand(3, n, lu + ld + 1), torch.rand(3, n, lu + ld + 1))

    def run(dev, dtype):
        s1 = band.to(dev, dtype).clone().requires_grad_(True)
        s2 = band2.to(dev, dtype).clone().requires_grad_(True)
        bk = back.to(dev, dtype).clone().requires_grad_(True)
        if dev.type == "cuda":
            out = BandedMatrix(s2, lu, ld).multiply_log(BandedMatrix(s1, lu, ld).transpose()).data
        else:  # dense closed form, float64 (test_sparse.py:181-195)
            X = BandedMatrix(BandedMatrix(s1, lu, ld).transpose().data, ld, lu, -1e9).to_dense()
            Y = BandedMatrix(s2, lu, ld, -1e9).to_dense()
            D = (X.transpose(-2, -1).unsqueeze(-1) + Y.unsqueeze(-3)).logsumexp(-2)
            out = banddiag(D, lu + lu, ld + ld)[0]
        g = torch.autograd.grad(out, (s1, s2), bk, create_graph=True)
        h = torch.autograd.grad((g[0], g[1]), (s1, s2, bk), (back2[0].to(dev, dtype), back2[1].to(dev, dtype)))
        return out, g, h

    out, g, h = run(gpu, torch.float32)
    wout, wg, wh = run(torch.device("cpu"), torch.float64)
    n_ = band.shape[1]
    mask = oracle.band_from_dense(torch.ones(1, n_, n_), 2 * lu, 2 * ld)[0] > 0
    close(out[:, mask.to(gpu)], wout[:, mask])
    assert bool((out[:, ~mask.to(gpu)] == 0).all())
    for x, y in zip(g, wg):
        close(x, y)
    for x, y in zip(h, wh):
        close(x, y, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", BANDS[:6])
def test_banded_double_backward_vs_literal_kernels(gpu, n, a_lu, a_ld, b_lu, b_ld):
    torch.manual_seed(n)
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld)
    W = a.shape[2] + b.shape[2] - 1
    g, u = torch.randn(3, n, W), torch.randn(*a.shape)
    want = oracle.seq_band_bwdbwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, g.double(), u.double(),
                                  dtype=np.float64)
    ad, bd, gd = (t.to(gpu).requires_grad_(True) for t in (a, b, g))
    out = BandedMatrix(ad, a_lu, a_ld).multiply_log(BandedMatrix(bd, b_lu, b_ld)).data
    (ga,) = torch.autograd.grad(out, (ad,), gd, create_graph=True)
    got = torch.autograd.grad(ga, (ad, bd, gd), u.to(gpu))
    for x, y in zip(got, want):
        close(x, y, rtol=1e-4, atol=1e-5)


def test_double_backward_reaches_operands_given_as_views(gpu):
    """Band tensors that are views (here: slices of wider tensors) are copied by a
    differentiable operation, so the second-order gradient with respect to the tensor
    the caller owns is complete - checked against float64 autograd through the dense
    closed form (test_sparse.py:181-195), and through the Function called directly."""
    from genbmm_amd.sparse import bandedlogbmm
    torch.manual_seed(21)
    n, a_lu, a_ld, b_lu, b_ld = 14, 2, 3, 1, 2
    wide_a, wide_b = torch.randn(2, n, 9), torch.randn(2, n, 8)   # operands: columns 1..6 and 2..5
    u = torch.randn(2, n, a_lu + a_ld + 1)

    def run(dev, dtype, direct=False):
        wa = wide_a.to(dev, dtype).requires_grad_(True)
        wb = wide_b.to(dev, dtype).requires_grad_(True)
        a, b = wa[:, :, 1:7], wb[:, :, 2:6]
        assert not a.is_contiguous()
        if dev.type == "cuda" and direct:
            out = bandedlogbmm(a, a_lu, a_ld, b, b_lu, b_ld, a_lu + b_ld, a_ld + b_lu)
        elif dev.type == "cuda":
            out = BandedMatrix(a, a_lu, a_ld).multiply_log(BandedMatrix(b, b_lu, b_ld)).data
        else:
            X = BandedMatrix(a, a_lu, a_ld, -1e9).to_dense()
            Y = BandedMatrix(b, b_lu, b_ld, -1e9).to_dense()
            D = (Y.transpose(-2, -1).unsqueeze(-1) + X.unsqueeze(-3)).logsumexp(-2)
            out = banddiag(D, a_lu + b_ld, a_ld + b_lu)[0]
        mask = oracle.band_from_dense(torch.ones(1, n, n), a_lu + b_ld, a_ld + b_lu)[0].to(dev) > 0
        g = torch.cos(torch.arange(out.numel(), device=dev, dtype=dtype)).reshape(out.shape) * mask
        (ga,) = torch.autograd.grad(out, a, g, create_graph=True)
        return torch.autograd.grad((ga * u.to(dev, dtype)).sum(), (wa, wb))

    want = run(torch.device("cpu"), torch.float64)
    for direct in (False, True):
        got = run(gpu, torch.float32, direct)
        for x, y in zip(got, want):
            assert float(y.abs().max()) > 0
            close(x, y, rtol=1e-4, atol=1e-5)


def test_banded_config_c5(gpu):
    """Benchmark configuration 4: batch 64, n = 4096, lu = ld = 32 for both operands, Uniform[-1,1)
    band data from seed 7; standard, log and max semiring, forward + backward, at full size.
    EVERY batch item: out, grad_a and grad_b against the float64 closed form over the cells'
    factor pairs (oracle.band_product64 and its autograd gradients, evaluated on the device
    item by item); the max product bit-exact (values, lowest-k indices, one-hot gradients with
    g on the 1/8 grid); two items against the sequential float64 restatement of the
    reference kernel; the dense closed form at reduced n."""
    torch.manual_seed(7)
    B, n, lu, ld = 64, 4096, 32, 32
    a, b = torch.rand(B, n, 65) * 2 - 1, torch.rand(B, n, 65) * 2 - 1
    g = torch.randn(B, n, 129)
    ad, bd, gd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True), g.to(gpu)
    pick = [0, 63]
    # absolute bound of a K-term fp32 sum against float64: 4 u K max|x| max|y| (u = 2^-24; the
    # textbook K u sum|x y| with room for the order of summation); the log product's
    # weights are at most 1, so its gradients obey the same bound with |y| = 1
    u, K = 2.0 ** -24, 65
    fwd_tol = 4 * u * K * float(a.abs().max()) * float(b.abs().max())
    bwd_tol = 4 * u * K * float(g.abs().max()) * max(float(a.abs().max()), float(b.abs().max()))
    assert fwd_tol < 2e-5 and bwd_tol < 1e-4
    for mode in (3, 0):
        X, Y = BandedMatrix(ad, lu, ld), BandedMatrix(bd, lu, ld)
        res = (X.multiply if mode == 3 else X.multiply_log)(Y)
        ga, gb = torch.autograd.grad(res.data, (ad, bd), gd)
        want, _, _ = oracle.seq_band_fwd(a[pick].double(), lu, ld, b[pick].double(), lu, ld, mode, dtype=np.float64)
        close(res.data[pick], want, rtol=1e-5, atol=fwd_tol)
        wa, wb = oracle.seq_band_bwd(a[pick].double(), lu, ld, b[pick].double(), lu, ld, g[pick].double(), mode,
                                     dtype=np.float64)
        close(ga[pick], wa, rtol=1e-5, atol=bwd_tol)
        close(gb[pick], wb, rtol=1e-5, atol=bwd_tol)
        for item in range(B):
            sl = slice(item, item + 1)
            a64 = ad[sl].detach().double().requires_grad_(True)
            b64 = bd[sl].detach().double().requires_grad_(True)
            w = oracle.band_product64(a64, lu, ld, b64, lu, ld, mode)
            wa, wb = torch.autograd.grad(w, (a64, b64), gd[sl].double())
            for got, ref, tol in ((res.data[sl].detach(), w.detach(), fwd_tol), (ga[sl], wa, bwd_tol), (gb[sl], wb, bwd_tol)):
                assert torch.allclose(got.double(), ref, rtol=1e-5, atol=tol), (mode, item, float((got.double() - ref).abs().max()))
            del w, wa, wb, a64, b64
    # max product, every item, bit for bit
    torch.manual_seed(8)
    aq, bq = grid(B, n, 65).to(gpu).requires_grad_(True), grid(B, n, 65).to(gpu).requires_grad_(True)
    gq = grid(B, n, 129).clamp(-4, 4).to(gpu)
    res = BandedMatrix(aq, lu, ld).multiply_max(BandedMatrix(bq, lu, ld))
    ga, gb = torch.autograd.grad(res.data, (aq, bq), gq)
    i = torch.arange(n, device=gpu).view(n, 1)
    jj = torch.arange(129, device=gpu).view(1, 129)
    o = i + jj - (lu + ld)
    inside = (o >= 0) & (o < n)
    for item in range(B):
        sl = slice(item, item + 1)
        mv, mi = oracle.band_max_first(aq[sl].detach(), lu, ld, bq[sl].detach(), lu, ld)
        assert torch.equal(res.data[sl].detach(), mv), item
        li = mi[0].long()
        wa = torch.zeros(n, 65, device=gpu).index_put_((i.expand(n, 129)[inside], li[inside]), gq[item][inside], accumulate=True)
        wb = torch.zeros(n, 65, device=gpu).index_put_((o[inside], (li - jj + 64)[inside]), gq[item][inside], accumulate=True)
        assert torch.equal(ga[item], wa) and torch.equal(gb[item], wb), item
    # dense closed form at n = 256, same bandwidths (test_sparse.py:141-142, 181-195)
    n2 = 256
    a2, b2 = a[:4, :n2].contiguous(), b[:4, :n2].contiguous()
    for mode in (3, 0):
        want, mask = oracle.band_product_dense(a2.double(), lu, ld, b2.double(), lu, ld, mode)
        X, Y = BandedMatrix(a2.to(gpu), lu, ld), BandedMatrix(b2.to(gpu), lu, ld)
        res = (X.multiply if mode == 3 else X.multiply_log)(Y)
        close(res.data[:, mask.to(gpu)], want[:, mask], rtol=1e-5, atol=4 * 2.0 ** -24 * 65)


def test_banded_errors(gpu):
    a = torch.randn(2, 5, 3)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        BandedMatrix(a, 1, 1).multiply(BandedMatrix(a, 1, 1))
    with pytest.raises(RuntimeError, match="disagree"):
        BandedMatrix(a.to(gpu), 1, 1).multiply_log(BandedMatrix(torch.randn(3, 5, 3, device=gpu), 1, 1))


@pytest.mark.parametrize("case", range(4))
def test_banded_products_match_reference_cpu_vectors(gpu, case):
    """Outputs of the reference's own CPU loops (sparse.py:268-401), stored by
    tests/golden/make_band_struct_fixtures.py: max is bit-exact, (+,x) and log to fp32
    rounding (the GPU sums with fused multiply-adds / in factored form)."""
    import os

    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "band_struct.npz"),
                allow_pickle=False)
    p = "c%d_" % case
    B, n, lu, ld, olu, old = (int(v) for v in z[p + "meta"])
    a = BandedMatrix(torch.from_numpy(z[p + "zband"]).to(gpu), lu, ld)
    b = BandedMatrix(torch.from_numpy(z[p + "zoband"]).to(gpu), olu, old)
    for fn, name, exact in ((a.multiply, "multiply_simple", False), (a.multiply_log, "multiply_log_simple", False),
                            (a.multiply_max, "multiply_max_simple", True)):
        got = fn(b)
        want = torch.from_numpy(z[p + name])
        assert [got.lu, got.ld] == [int(v) for v in z[p + name + "_luld"]]
        if exact:
            assert torch.equal(got.data.cpu(), want), name
        else:
            assert torch.allclose(got.data.cpu(), want, rtol=1e-5, atol=1e-5), name


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", BANDS)
def test_banded_log_without_workspace(gpu, n, a_lu, a_ld, b_lu, b_ld):
    """The log product through the C ABI with workspace = NULL (every exponential taken
    in the strip kernels) against the float64 oracle; the Python layer always passes a
    workspace, so this is the only caller of that path."""
    lib = _lib.load()
    torch.manual_seed(n + a_lu)
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld)
    W = a.shape[2] + b.shape[2] - 1
    g = torch.randn(3, n, W)
    ad, bd, gd = a.to(gpu), b.to(gpu), g.to(gpu)
    out, ga, gb = torch.empty(3, n, W, device=gpu), torch.empty_like(ad), torch.empty_like(bd)
    p, s, null = _lib.ptr, _lib.stream_of(ad), _lib.ptr(None)
    assert lib.genbmm_banded_fwd(p(ad), a_lu, a_ld, p(bd), b_lu, b_ld, p(out), null, null, 3, n, 0, s) == 0
    assert lib.genbmm_banded_bwd(p(ad), a_lu, a_ld, p(bd), b_lu, b_ld, p(out), null, null, p(gd), p(ga), p(gb),
                                 3, n, 0, s) == 0
    want, _, _ = oracle.seq_band_fwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, 0, dtype=np.float64)
    wa, wb = oracle.seq_band_bwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, g.double(), 0, dtype=np.float64)
    close(out, want)
    close(ga, wa)
    close(gb, wb)


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", [(70, 3, 5, 4, 2), (150, 14, 13, 12, 15), (64, 8, 8, 8, 8),
                                                   (70, 1, 0, 4, 2), (90, 0, 1, 1, 0)])
def test_backward_with_separate_scratch_leaves_the_workspace_alone(gpu, n, a_lu, a_ld, b_lu, b_ld):
    """genbmm_banded_bwd_scratch: same gradients as genbmm_banded_bwd, bit for bit, and the
    workspace the forward filled is not written."""
    lib = _lib.load()
    torch.manual_seed(n)
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld)
    B, W = 3, a.shape[2] + b.shape[2] - 1
    ad, bd, g = a.to(gpu), b.to(gpu), torch.randn(B, n, W).to(gpu)
    out = torch.empty(B, n, W, device=gpu)
    ws = torch.zeros(lib.genbmm_banded_workspace_size(a_lu, a_ld, b_lu, b_ld, B, n), device=gpu)
    s, p = _lib.stream_of(ad), _lib.ptr
    assert lib.genbmm_banded_fwd(p(ad), a_lu, a_ld, p(bd), b_lu, b_ld, p(out), p(None), p(ws), B, n, 0, s) == 0
    before = ws.clone()
    need = lib.genbmm_banded_scratch_size(a_lu, a_ld, b_lu, b_ld, B, n)
    assert need in (0, B * n * W)
    scratch = torch.empty(need, device=gpu) if need else None
    ga, gb = torch.empty_like(ad), torch.empty_like(bd)
    assert lib.genbmm_banded_bwd_scratch(p(ad), a_lu, a_ld, p(bd), b_lu, b_ld, p(out), p(None), p(ws), p(scratch),
                                         p(g), p(ga), p(gb), B, n, 0, s) == 0
    assert torch.equal(ws, before)
    wa, wb = torch.empty_like(ad), torch.empty_like(bd)
    assert lib.genbmm_banded_bwd(p(ad), a_lu, a_ld, p(bd), b_lu, b_ld, p(out), p(None), p(ws), p(g), p(wa), p(wb),
                                 B, n, 0, s) == 0
    assert torch.equal(ga, wa) and torch.equal(gb, wb)
    # a workspace without the scratch it needs is refused; the other modes take neither
    if need:
        assert lib.genbmm_banded_bwd_scratch(p(ad), a_lu, a_ld, p(bd), b_lu, b_ld, p(out), p(None), p(ws), p(None),
                                             p(g), p(ga), p(gb), B, n, 0, s) != 0
    assert lib.genbmm_banded_bwd_scratch(p(ad), a_lu, a_ld, p(bd), b_lu, b_ld, p(None), p(None), p(None), p(None),
                                         p(g), p(ga), p(gb), B, n, 3, s) == 0
    assert lib.genbmm_banded_bwd(p(ad), a_lu, a_ld, p(bd), b_lu, b_ld, p(None), p(None), p(None), p(g), p(wa), p(wb),
                                 B, n, 3, s) == 0
    assert torch.equal(ga, wa) and torch.equal(gb, wb)
