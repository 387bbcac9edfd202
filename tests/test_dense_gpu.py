"""GPU parity of the dense semiring ops against the CPU oracle (all marked gpu).

Tolerances: logbmm forward / gradients rtol 1e-5, atol 1e-5 against float64;
max / prod-max values, indices and gradients bit-exact; sampling by a CDF
bracket check per cell plus a chi-square bound.
"""
import ctypes
import math

import numpy as np
import pytest
import torch

import oracle
import genbmm_amd as genbmm
from genbmm_amd import _lib, genmul

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-5


def close(x, ref, rtol=RTOL, atol=ATOL):
    x, ref = x.detach().cpu().double(), ref.detach().cpu().double()
    bad = ~torch.isclose(x, ref, rtol=rtol, atol=atol, equal_nan=True)
    if bad.any():
        err = (x - ref).abs()
        raise AssertionError("max abs err %.3e over %d cells, worst at %s" % (
            float(err[bad].max()), int(bad.sum()), np.unravel_index(int(err.argmax()), x.shape)))


def lse64(a, b, chunk=4):
    outs = [oracle.logbmm_broadcast(a[i:i + chunk].double(), b[i:i + chunk].double())
            for i in range(0, a.shape[0], chunk)]
    return torch.cat(outs) if outs else a.new_zeros((0, a.shape[1], b.shape[2])).double()


@pytest.fixture(params=["factored", "exact", "factored-valu", "factors-kept", "fp32-matrix"])
def path(request, gpu):
    """Run a logbmm test on every kernel family of the library: the default one (whole-item
    kernels for small matrices, matrix cores for large ones, factored vector-ALU kernels
    between; the matrix-core kernels keep the maxima only and form their operands again in the
    backward), the online / exact kernels alone, the factored kernels on v_fma only, and the
    default kernels with the forward's factors kept for an exponent-free backward, and the default
    kernels with the fp32 matrix instruction wherever the default uses the bf16 one on three-part
    factors.  The value is the `path` argument of genbmm_logbmm_fwd_path / _bwd_path."""
    return {"factored": genmul.PATH_AUTO, "exact": genmul.PATH_EXACT, "factored-valu": genmul.PATH_VALU,
            "factors-kept": genmul.PATH_FACTORS, "fp32-matrix": genmul.PATH_MFMA32}[request.param]


def logbmm_on(path):
    return lambda a, b: genmul.logbmm_on_path(a, b, path)


SHAPES = [(16, 64, 64, 64), (3, 7, 9, 5), (2, 1, 1, 1), (4, 5, 1, 6), (5, 33, 70, 129), (2, 130, 17, 66),
          (3, 64, 64, 128), (2, 200, 96, 260), (9, 32, 32, 32), (7, 31, 33, 29), (1, 256, 40, 256),
          (6, 128, 128, 128), (11, 100, 70, 128), (3, 65, 64, 64), (9, 127, 99, 101)]


@pytest.mark.parametrize("B,M,K,N", SHAPES)
def test_logbmm_forward_and_grads(gpu, path, B, M, K, N):
    torch.manual_seed(B * 1000 + M)
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    want, wa, wb = oracle.logbmm_grads64(a, b, g)
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = logbmm_on(path)(ad, bd)
    close(out, want)
    ga, gb = torch.autograd.grad(out, (ad, bd), g.to(gpu))
    close(ga, wa)
    close(gb, wb)
    # softmax weights sum to one over k
    close(ga.sum(-1), g.double().sum(-1), atol=1e-4)
    close(gb.sum(-2), g.double().sum(-2), atol=1e-4)


def test_logbmm_config_c1_uniform_ones(gpu, path):
    """Benchmark configuration 0: seed 0, Uniform[0,1) (16,64,64), grad_out = ones."""
    torch.manual_seed(0)
    a, b = torch.rand(16, 64, 64), torch.rand(16, 64, 64)
    g = torch.ones(16, 64, 64)
    want, wa, wb = oracle.logbmm_grads64(a, b, g)
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = logbmm_on(path)(ad, bd)
    ga, gb = torch.autograd.grad(out.sum(), (ad, bd))
    close(out, want)
    close(ga, wa)
    close(gb, wb)
    # the sequential fp32 restatement of the reference kernel agrees too
    close(out, oracle.seq_logbmm_fwd(a, b)[0])


def test_logbmm_special_values(gpu, path):
    a, b = torch.randn(2, 5, 6), torch.randn(2, 6, 4)
    b[0, 2, :] = -math.inf          # masked k
    a[1, 3, :] = -math.inf          # fully masked row -> -inf
    a[0, 1, :] = -2e9               # below the -1e9 floor -> -inf, as in the reference
    got = logbmm_on(path)(a.to(gpu), b.to(gpu)).cpu()
    want, _ = oracle.seq_logbmm_fwd(a, b)
    assert torch.equal(torch.isinf(got), torch.isinf(want))
    fin = ~torch.isinf(want)
    close(got[fin], want[fin])
    big = torch.randn(2, 9, 33) * 30 + 200  # large magnitudes
    bb = torch.randn(2, 33, 7) * 30 - 500
    close(logbmm_on(path)(big.to(gpu), bb.to(gpu)), lse64(big, bb))
    a1, b1 = torch.randn(2, 5, 1), torch.randn(2, 1, 4)               # K = 1: out = a + b
    close(logbmm_on(path)(a1.to(gpu), b1.to(gpu)), a1 + b1, rtol=1e-6, atol=1e-6)


def close_on_device(x, ref, what, rtol=RTOL, atol=ATOL):
    """`close` without leaving the device (full-size tensors): x, ref on the GPU, ref float64."""
    bad = ~torch.isclose(x.double(), ref, rtol=rtol, atol=atol, equal_nan=True)
    if bool(bad.any()):
        err = (x.double() - ref).abs()
        raise AssertionError("%s: max abs err %.3e over %d cells, worst at %s" % (
            what, float(err[bad].max()), int(bad.sum()), np.unravel_index(int(err.argmax()), tuple(x.shape))))


@pytest.mark.parametrize("B,M,K,N,chunk", [(512, 128, 128, 128, 64), (8192, 32, 32, 32, 2048), (64, 512, 512, 512, 1)])
def test_logbmm_baseline_shapes(gpu, path, B, M, K, N, chunk):
    """Benchmark configuration 1 and the headline shape at full size: out, grad_a and grad_b of
    EVERY batch item against the float64 closed form (the broadcast log-sum-exp and its
    autograd gradients, evaluated on the device `chunk` items at a time - 1 GiB of float64
    terms per step), plus the size-independent row-sum invariants."""
    torch.manual_seed(0)
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    ad, bd, gd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True), g.to(gpu)
    out = logbmm_on(path)(ad, bd)
    ga, gb = torch.autograd.grad(out, (ad, bd), gd)
    for i in range(0, B, chunk):
        sl = slice(i, i + chunk)
        want, wa, wb = oracle.logbmm_grads64(ad[sl], bd[sl], gd[sl])
        close_on_device(out[sl].detach(), want, "out, items %d.." % i)
        close_on_device(ga[sl], wa, "grad_a, items %d.." % i)
        close_on_device(gb[sl], wb, "grad_b, items %d.." % i)
        del want, wa, wb
    close(ga.sum(-1), gd.double().sum(-1), atol=2e-4)
    close(gb.sum(-2), gd.double().sum(-2), atol=2e-4)
    # out >= max_k(a+b) and out <= max + log K
    mx = genbmm.maxbmm(ad.detach(), bd.detach())
    assert bool((out >= mx - 1e-5).all()) and bool((out <= mx + math.log(K) + 1e-5).all())


@pytest.mark.parametrize("B,M,K,N", [(2, 40, 48, 36), (3, 130, 64, 140), (2, 256, 32, 256), (5, 32, 32, 32)])
def test_logbmm_factoring_guard(gpu, B, M, K, N):
    """Inputs for which exp(a - rowmax) * exp(b - colmax) underflows although the true
    terms do not: the factored kernels must detect it per tile and fall back."""
    torch.manual_seed(B + M)
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    # every second row of a peaks at k = 0 while b's row 0 is 200 below the rest
    a[:, ::2, 0] += 200.0
    b[:, 0, :] -= 200.0
    # one batch item carries -2e9 masks on disjoint halves of k: every term is below the
    # -1e9 floor -> -inf (matmul_cuda_kernel.cu:31-41)
    a[-1, :, ::2] = -2e9
    b[-1, 1::2, :] = -2e9
    want, wa, wb = oracle.logbmm_grads64(a[:-1], b[:-1], g[:-1])
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = genbmm.logbmm(ad, bd)
    close(out[:-1], want)
    ref32, _ = oracle.seq_logbmm_fwd(a[-1:], b[-1:])
    assert bool(torch.isinf(ref32).all()) and bool(torch.isinf(out[-1]).all())
    ga, gb = torch.autograd.grad(out[:-1].sum() * 0 + (out[:-1] * g[:-1].to(gpu)).sum(), (ad, bd))
    close(ga[:-1], wa)
    close(gb[:-1], wb)
    # the two paths agree with each other on these inputs as well
    out2 = genmul.logbmm_on_path(ad, bd, genmul.PATH_EXACT)
    ga2, gb2 = torch.autograd.grad((out2[:-1] * g[:-1].to(gpu)).sum(), (ad, bd))
    close(out2[:-1], want)
    close(ga2[:-1], wa)
    close(gb2[:-1], wb)


@pytest.mark.parametrize("B,M,K,N", [(32, 256, 128, 256), (64, 512, 128, 512), (64, 200, 100, 260),
                                     (64, 500, 132, 500), (128, 260, 388, 132), (24, 201, 103, 259),
                                     (3, 130, 97, 391), (64, 257, 255, 129)])
@pytest.mark.parametrize("keep", [False, True])
def test_logbmm_factoring_guard_matrix_core_tiles(gpu, keep, B, M, K, N):
    """Shapes that run on the matrix-core kernels (128x128 and 128x256 / 256x128 tiles),
    all but the first two with ragged edges in every dimension (partial tiles, partial slabs),
    the last three with odd sizes (rows not 16-byte aligned, pieces straddling the edge).
    Some batch items need the exact fall-back in every tile, one in a single row, the
    rest in none: flagged and unflagged tiles side by side, and the backward kernels
    must honour the forward's flags.  keep: the forward's factors are kept and the backward
    reads 1/S from the workspace (GENBMM_PATH_FACTORS); else only the maxima are kept and the
    backward forms its operands again."""
    torch.manual_seed(B + M)
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    a[: B // 4, ::2, 0] += 200.0
    b[: B // 4, 0, :] -= 200.0
    a[B // 4, 37, 5] += 200.0
    b[B // 4, 5, :] -= 200.0
    pick = torch.tensor([0, 1, B // 4, B // 4 + 1, B - 1])
    want, wa, wb = oracle.logbmm_grads64(a[pick], b[pick], g[pick])
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = genmul.logbmm_on_path(ad, bd, genmul.PATH_FACTORS) if keep else genbmm.logbmm(ad, bd)
    ga, gb = torch.autograd.grad(out, (ad, bd), g.to(gpu))
    close(out[pick.to(gpu)], want)
    close(ga[pick.to(gpu)], wa)
    close(gb[pick.to(gpu)], wb)
    close(ga.sum(-1), g.double().sum(-1), atol=2e-4)
    close(gb.sum(-2), g.double().sum(-2), atol=2e-4)


@pytest.mark.parametrize("B,M,K,N", [(8, 256, 128, 256), (6, 300, 100, 260), (4, 512, 64, 384), (9, 32, 32, 32),
                                     (6, 64, 64, 64), (5, 40, 48, 36), (7, 128, 128, 128), (4, 100, 70, 128)])
@pytest.mark.parametrize("keep", [False, True])
def test_logbmm_rows_masked_at_the_floor(gpu, keep, B, M, K, N):
    """Padding written as -1e9, the reference's own floor (matmul_cuda_kernel.cu:31): whole
    rows of a, whole columns of b, or - one batch item - both.  A cell of a masked row has
    max_k(a + b) = -1e9 + max_k b, not below the floor, so the reference's result is the
    plain log-sum-exp there (float64: -1e9 + logsumexp_k b[k, n]; a float holds it to within
    64); where a masked row meets a masked column every term is at -2e9 and the reference
    gives -inf.  The gradient flowing into the padding is zero, as after any masked loss;
    the gradients of everything else must not notice the padding.  On the matrix-core shapes
    the tiles with masked rows or columns are factored like any other (their 1 / S comes from
    the sums, not from `out`), only the tiles of the item with both take the exact routine;
    the smaller shapes run the whole-item kernels, the factored vector-ALU kernels and the
    one-tile-per-item kernels (whose padded items take the exact routine)."""
    torch.manual_seed(B + N)
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    rows, cols = M - M // 5, N - N // 7
    a[: B // 2, rows:, :] = -1e9          # padded rows
    b[B // 2:, :, cols:] = -1e9           # padded columns
    a[B - 1, rows:, :] = -1e9             # the last item: both
    g[: B // 2, rows:, :] = 0.0
    g[B // 2:, :, cols:] = 0.0
    g[B - 1, rows:, :] = 0.0
    want, wa, wb = oracle.logbmm_grads64(a, b, g)
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = genmul.logbmm_on_path(ad, bd, genmul.PATH_FACTORS) if keep else genbmm.logbmm(ad, bd)
    ga, gb = torch.autograd.grad(out, (ad, bd), g.to(gpu))
    both = torch.zeros(B, M, N, dtype=torch.bool)
    both[B - 1, rows:, cols:] = True
    pad = torch.zeros(B, M, N, dtype=torch.bool)
    pad[: B // 2, rows:, :] = True
    pad[B // 2:, :, cols:] = True
    pad[B - 1, rows:, :] = True
    pad &= ~both
    oc = out.cpu()
    assert bool(torch.isinf(oc[both]).all()) and bool((oc[both] < 0).all())
    close(oc[~pad & ~both], want[~pad & ~both])
    close(oc[pad], want[pad], rtol=0, atol=128.0)   # a float near -1e9 is a multiple of 64
    # the exact routine and the factored vector-ALU kernels (the reference's own steps at the padding) agree
    for other in (genmul.PATH_EXACT, genmul.PATH_VALU):
        alt = genmul.logbmm_on_path(ad.detach(), bd.detach(), other).cpu()
        assert torch.equal(torch.isinf(alt), torch.isinf(oc))
        close(oc[~pad & ~both], alt[~pad & ~both])
        close(oc[pad], alt[pad], rtol=0, atol=128.0)
    # gradients: the item with both has infinite weights where the reference has them (0 * inf);
    # the others are finite everywhere and equal to float64's
    ok = torch.arange(B) != B - 1
    close(ga[ok.to(gpu)], wa[ok])
    close(gb[ok.to(gpu)], wb[ok])
    assert bool(torch.isfinite(ga[ok.to(gpu)]).all()) and bool(torch.isfinite(gb[ok.to(gpu)]).all())


@pytest.mark.parametrize("B,M,K,N", [(64, 512, 256, 512), (64, 512, 512, 384), (64, 512, 512, 512), (48, 768, 64, 512),
                                     (64, 500, 300, 500), (64, 500, 500, 300), (64, 509, 253, 499), (64, 1000, 250, 300),
                                     (64, 496, 500, 496), (64, 496, 508, 304), (40, 1008, 252, 400)])
def test_logbmm_three_part_kernels(gpu, B, M, K, N):
    """Shapes which the default path runs on the bf16 matrix instruction with
    every factor cut into three bf16 parts (256 x 256 tiles where they fill the chip, 256 x 128 /
    128 x 256 otherwise; forward and backward switch independently; the last seven with ragged
    edges - partial tiles, partial slabs, odd row lengths; the backward takes any M, and K and N in
    multiples of four): every batch item against
    float64 on the device, among them items whose tiles must take the exact routine (factors that
    underflow against live terms: everywhere, and in a single row), an item with rows padded at
    the floor, one with a masked reduction step, one with magnitudes near 1000 - and the whole
    result against the fp32 matrix instruction (GENBMM_PATH_MFMA32) at twice the tolerance."""
    torch.manual_seed(M + N)
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    a[1, ::2, 0] += 200.0
    b[1, 0, :] -= 200.0
    a[2, 37, 5] += 200.0
    b[2, 5, :] -= 200.0
    a[3, M - 50:, :] = -1e9
    g[3, M - 50:, :] = 0.0
    a[4] *= 300.0
    b[5, 7, :] = -float("inf")
    ad, bd, gd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True), g.to(gpu)
    out = genbmm.logbmm(ad, bd)
    ga, gb = torch.autograd.grad(out, (ad, bd), gd)
    for i in range(B):
        want, wa, wb = oracle.logbmm_grads64(ad[i:i + 1], bd[i:i + 1], gd[i:i + 1])
        rows = slice(0, M - 50) if i == 3 else slice(0, M)   # the padded rows' own cells: rounding artefacts
        # (item 4: `out` near 1000 is rounded to 6e-5, and every backward that forms its weights from
        #  `out` - the reference's included - inherits that as a relative error of the weights)
        tol = dict(rtol=1e-3, atol=5e-3) if i == 4 else {}
        close_on_device(out[i:i + 1, rows].detach(), want[:, rows], "out, item %d" % i)
        close_on_device(ga[i:i + 1, rows], wa[:, rows], "grad_a, item %d" % i, **tol)
        close_on_device(gb[i:i + 1], wb, "grad_b, item %d" % i, **tol)
        del want, wa, wb
    assert bool(torch.isfinite(ga).all()) and bool(torch.isfinite(gb).all())
    ar, br = ad.detach().clone().requires_grad_(True), bd.detach().clone().requires_grad_(True)
    ref = genmul.logbmm_on_path(ar, br, genmul.PATH_MFMA32)
    ra, rb = torch.autograd.grad(ref, (ar, br), gd)
    keep = torch.ones(M, dtype=torch.bool, device=gpu)
    for x, y, rowwise, grad in ((out.detach(), ref.detach(), True, False), (ga, ra, True, True), (gb, rb, False, True)):
        x, y = x.clone(), y.clone()
        if rowwise:   # item 3's padded rows again
            x[3, M - 50:], y[3, M - 50:] = 0, 0
        if grad:
            close_on_device(x[4], y[4].double(), "item 4 against the fp32 matrix instruction", rtol=1e-3, atol=5e-3)
            x[4], y[4] = 0, 0
        close_on_device(x, y.double(), "against the fp32 matrix instruction", rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("B,M,K,N,scale", [(64, 512, 512, 512, 1.0), (8, 1024, 2048, 512, 1.0), (32, 500, 1000, 400, 3.0),
                                            (512, 128, 128, 128, 1.0)])
def test_three_part_products_are_as_accurate_as_fp32_products(gpu, B, M, K, N, scale):
    """The default kernels take every product as six bf16 partial products of three-part factors;
    GENBMM_PATH_MFMA32 takes it on the fp32 matrix instruction.  Against float64 (four batch items,
    on the device) the two must be equally good: maximum and mean absolute error of out, grad_a
    and grad_b on the default path at most 1.5 times the fp32 instruction's (+ 1e-7)."""
    torch.manual_seed(K)
    a, b, g = (torch.randn(B, M, K, device=gpu) * scale, torch.randn(B, K, N, device=gpu) * scale,
               torch.randn(B, M, N, device=gpu))
    pick = slice(0, 4)
    want = oracle.logbmm_grads64(a[pick], b[pick], g[pick])
    errs = []
    for path in (genmul.PATH_AUTO, genmul.PATH_MFMA32):
        ad, bd = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
        out = genmul.logbmm_on_path(ad, bd, path)
        res = (out.detach(),) + torch.autograd.grad(out, (ad, bd), g)
        errs.append([((x[pick].double() - w).abs().max().item(), (x[pick].double() - w).abs().mean().item())
                     for x, w in zip(res, want)])
    for (mx3, mean3), (mx32, mean32), what in zip(errs[0], errs[1], ("out", "grad_a", "grad_b")):
        assert mx3 <= 1.5 * mx32 + 1e-7, (what, mx3, mx32)
        assert mean3 <= 1.5 * mean32 + 1e-7, (what, mean3, mean32)


def test_logbmm_matrix_core_shape_sweep(gpu):
    """A seeded sweep of 48 shapes around the switching points of the matrix-core kernels (tile forms
    256 x 256 / 256 x 128 / 128 x 128, full and ragged, extents in multiples of 16, of 4 and odd -
    the backward takes the bf16 instruction for K and N in multiples of four, else the fp32 one):
    the default path against float64 on the device, and against GENBMM_PATH_MFMA32."""
    rng = np.random.RandomState(7)
    shapes = []
    for i in range(48):
        step = (16, 4, 1)[i % 3]
        M, K, N = (int(rng.randint(96 // step, 700 // step + 1)) * step for _ in range(3))
        B = int(rng.choice([1, 3, 8, 24, 64]))
        if B * M * N > 64 * 512 * 512:
            B = max(1, (64 * 512 * 512) // (M * N))
        shapes.append((B, M, K, N))
    shapes += [(64, 256, 96, 512), (24, 512, 16, 768), (5, 1024, 272, 256)]
    for B, M, K, N in shapes:
        torch.manual_seed(M * 7 + N)
        a, b, g = (torch.randn(B, M, K, device=gpu), torch.randn(B, K, N, device=gpu), torch.randn(B, M, N, device=gpu))
        res = []
        for path in (genmul.PATH_AUTO, genmul.PATH_MFMA32):
            ad, bd = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
            out = genmul.logbmm_on_path(ad, bd, path)
            res.append((out.detach(),) + torch.autograd.grad(out, (ad, bd), g))
        pick = slice(0, min(B, 4))
        want = oracle.logbmm_grads64(a[pick], b[pick], g[pick])
        for x, y, w, what in zip(res[0], res[1], want, ("out", "grad_a", "grad_b")):
            close_on_device(x[pick], w, "%s of %s" % (what, (B, M, K, N)))
            close_on_device(x, y.double(), "%s of %s against the fp32 matrix instruction" % (what, (B, M, K, N)),
                            rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("B,M,K,N", [(20, 128, 128, 128), (17, 100, 70, 128), (12, 64, 128, 65), (9, 127, 99, 101)])
def test_logbmm_one_tile_items(gpu, B, M, K, N):
    """Items of at most 128 in every extent: one workgroup per item (and gradient) that
    takes the maxima, the factors and the guard itself.  Items that need the exact routine
    (underflowing factors in every row, in one row, masked terms, a fully masked row) sit
    between items that do not; either gradient alone; a workspace another forward filled."""
    lib = _lib.load()
    torch.manual_seed(B + M)
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    a[1, ::2, 0] += 200.0
    b[1, 0, :] -= 200.0
    a[4, 37, 5] += 200.0
    b[4, 5, :] -= 200.0
    a[6, :, ::2] = -2e9   # every term of item 6 below the -1e9 floor -> -inf
    b[6, 1::2, :] = -2e9
    b[7, 3, :] = -math.inf  # one masked k
    fin = torch.tensor([i for i in range(B) if i != 6])
    want, wa, wb = oracle.logbmm_grads64(a[fin], b[fin], g[fin])
    ad, bd, gd = a.to(gpu), b.to(gpu), g.to(gpu)
    out, ga, gb = torch.empty(B, M, N, device=gpu), torch.empty_like(ad), torch.empty_like(bd)
    size = lib.genbmm_logbmm_stats_size(B, M, K, N)
    # maxima, one flag word per 32 x 32 cells, header: no copy of any operand
    assert size <= B * (M + N) + B * 16 + 8 and lib.genbmm_samplebmm_stats_size(B, M, K, N) >= size
    stats = torch.full((size,), float("nan"), device=gpu)
    p, s = _lib.ptr, _lib.stream_of(ad)
    assert lib.genbmm_logbmm_fwd(p(ad), p(bd), p(out), p(stats), B, M, K, N, s) == 0
    close(out[fin.to(gpu)], want)
    assert bool(torch.isinf(out[6]).all())
    # the maxima are in the workspace for the backward
    close(stats[: B * (M + N)].view(B, M + N)[:, :M], a.amax(-1), rtol=0, atol=0)
    close(stats[: B * (M + N)].view(B, M + N)[:, M:], b.amax(-2), rtol=0, atol=0)
    before = stats.clone()
    assert lib.genbmm_logbmm_bwd(p(ad), p(bd), p(out), p(gd), p(stats), p(ga), p(gb), B, M, K, N, s) == 0
    assert torch.equal(before.view(torch.int32), stats.view(torch.int32))  # the backward only reads it
    close(ga[fin.to(gpu)], wa)
    close(gb[fin.to(gpu)], wb)
    ok = torch.tensor([i for i in range(B) if i not in (6, 7)])
    close(ga[ok.to(gpu)].sum(-1), g[ok].double().sum(-1), atol=2e-4)
    close(gb[ok.to(gpu)].sum(-2), g[ok].double().sum(-2), atol=2e-4)
    # either gradient alone
    ga1, gb1 = torch.full_like(ad, 7.0), torch.full_like(bd, 7.0)
    assert lib.genbmm_logbmm_bwd(p(ad), p(bd), p(out), p(gd), p(stats), p(ga1), p(None), B, M, K, N, s) == 0
    assert lib.genbmm_logbmm_bwd(p(ad), p(bd), p(out), p(gd), p(stats), p(None), p(gb1), B, M, K, N, s) == 0
    assert torch.equal(ga1[fin.to(gpu)], ga[fin.to(gpu)]) and torch.equal(gb1[fin.to(gpu)], gb[fin.to(gpu)])
    # a workspace filled by the vector-ALU forward (same maxima, other tag), and one filled by
    # nothing at all (every item falls back to the exact routine)
    out2 = torch.empty_like(out)
    assert lib.genbmm_logbmm_fwd_path(p(ad), p(bd), p(out2), p(stats), B, M, K, N, genmul.PATH_VALU, s) == 0
    close(out2[fin.to(gpu)], want)
    ga2, gb2 = torch.empty_like(ad), torch.empty_like(bd)
    assert lib.genbmm_logbmm_bwd(p(ad), p(bd), p(out2), p(gd), p(stats), p(ga2), p(gb2), B, M, K, N, s) == 0
    close(ga2[fin.to(gpu)], wa)
    close(gb2[fin.to(gpu)], wb)
    stats.zero_()
    assert lib.genbmm_logbmm_bwd(p(ad), p(bd), p(out), p(gd), p(stats), p(ga2), p(gb2), B, M, K, N, s) == 0
    close(ga2[fin.to(gpu)], wa)
    close(gb2[fin.to(gpu)], wb)


def test_logbmm_backward_on_foreign_workspace(gpu):
    """The exponent-free matrix-core backward (GENBMM_PATH_FACTORS) runs on by-products of the
    matrix-core forward; handed a workspace that another forward path filled - the vector-ALU
    forward, or the default matrix-core forward, which keeps the maxima only - it must notice
    and still be right (every tile then goes to the exact routine).  The default backward takes
    any of them as they are."""
    lib = _lib.load()
    torch.manual_seed(3)
    B, M, K, N = 32, 256, 128, 256
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    ad, bd, gd = a.to(gpu), b.to(gpu), g.to(gpu)
    p, s = _lib.ptr, _lib.stream_of(ad)
    big = lib.genbmm_logbmm_stats_size_path(B, M, K, N, genmul.PATH_FACTORS)
    assert big > B * (M * K + K * N + M * N) > lib.genbmm_logbmm_stats_size(B, M, K, N)
    pick = torch.tensor([0, B - 1])
    want, wa, wb = oracle.logbmm_grads64(a[pick], b[pick], g[pick])
    for fwd_path in (genmul.PATH_VALU, genmul.PATH_AUTO, genmul.PATH_FACTORS):
        for bwd_path in (genmul.PATH_FACTORS, genmul.PATH_AUTO):
            out, ga, gb = torch.empty(B, M, N, device=gpu), torch.empty_like(ad), torch.empty_like(bd)
            stats = torch.full((big,), float("nan"), device=gpu)
            assert lib.genbmm_logbmm_fwd_path(p(ad), p(bd), p(out), p(stats), B, M, K, N, fwd_path, s) == 0
            before = stats.clone()
            assert lib.genbmm_logbmm_bwd_path(p(ad), p(bd), p(out), p(gd), p(stats), p(ga), p(gb), B, M, K, N, bwd_path, s) == 0
            assert torch.equal(before.view(torch.int32), stats.view(torch.int32))  # the backward only reads it
            close(out[pick.to(gpu)], want)
            close(ga[pick.to(gpu)], wa)
            close(gb[pick.to(gpu)], wb)
            close(ga.sum(-1), g.double().sum(-1), atol=2e-4)


@pytest.mark.parametrize("B,M,K,N", [(2, 4, 5, 3), (3, 9, 12, 7), (2, 33, 20, 40)])
def test_logbmm_double_backward(gpu, B, M, K, N):
    """Second-order terms (test_cuda.py:30-42 uses rtol 1e-2; here 1e-4 vs float64)."""
    torch.manual_seed(7)
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    ua, ub = torch.randn(B, M, K), torch.randn(B, K, N)
    for u_a, u_b in [(ua, ub), (ua, None), (None, ub)]:
        want = oracle.logbmm_second_order64(a, b, g, u_a, u_b)
        ad, bd, gd = (t.to(gpu).requires_grad_(True) for t in (a, b, g))
        out = genbmm.logbmm(ad, bd)
        ga, gb = torch.autograd.grad(out, (ad, bd), gd, create_graph=True)
        outs = [t for t, u in ((ga, u_a), (gb, u_b)) if u is not None]
        cots = [u.to(gpu) for u in (u_a, u_b) if u is not None]
        got = torch.autograd.grad(outs, (ad, bd, gd), cots)
        for x, y in zip(got, want):
            close(x, y, rtol=1e-4, atol=1e-5)
    # the reference's literal quartic kernels (u_b = 0), fp32 sequential
    qa, qb, qg = oracle.seq_logbmm_bwdbwd(a.double(), b.double(), g.double(), ua.double(), dtype=np.float64)
    want = oracle.logbmm_second_order64(a, b, g, ua, None)
    for x, y in zip((qa, qb, qg), want):
        close(x, y, rtol=1e-9, atol=1e-11)


def test_logbmm_double_backward_at_a_matrix_core_shape(gpu):
    """Second-order terms on a shape whose forward and backward run on the matrix cores
    ((8, 256, 128, 256): ragged nowhere, two 128-wide tiles a side), against float64
    autograd with create_graph on two of the batch items."""
    torch.manual_seed(17)
    B, M, K, N = 8, 256, 128, 256
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    ua, ub = torch.randn(B, M, K), torch.randn(B, K, N)
    ad, bd, gd = (t.to(gpu).requires_grad_(True) for t in (a, b, g))
    out = genbmm.logbmm(ad, bd)
    ga, gb = torch.autograd.grad(out, (ad, bd), gd, create_graph=True)
    got = torch.autograd.grad((ga, gb), (ad, bd, gd), (ua.to(gpu), ub.to(gpu)))
    pick = [1, 6]
    want = oracle.logbmm_second_order64(a[pick], b[pick], g[pick], ua[pick], ub[pick])
    for x, y in zip(got, want):
        # sums of up to 256 terms of magnitude |g u| <= ~20: absolute fp32 error well under 1e-4
        close(x[pick], y, rtol=1e-4, atol=1e-4)


def _bwdbwd_abi(gpu, a, b, out, g, u_a, u_b, use_ws):
    lib = _lib.load()
    B, M, K = a.shape
    N = b.shape[2]
    ga, gb, gg = torch.empty_like(a), torch.empty_like(b), torch.empty_like(g)
    p, s = _lib.ptr, _lib.stream_of(a)
    if use_ws:
        ws = torch.empty(lib.genbmm_logbmm_bwdbwd_ws_size(B, M, K, N), device=gpu)
        rc = lib.genbmm_logbmm_bwdbwd_ws(p(a), p(b), p(out), p(g), p(u_a), p(u_b), p(ga), p(gb), p(gg), p(ws), B, M, K, N, s)
    else:
        rc = lib.genbmm_logbmm_bwdbwd(p(a), p(b), p(out), p(g), p(u_a), p(u_b), p(ga), p(gb), p(gg), B, M, K, N, s)
    assert rc == 0
    return ga, gb, gg


@pytest.mark.parametrize("B,M,K,N", [(16, 128, 128, 128), (9, 100, 70, 130), (3, 200, 96, 260), (5, 64, 300, 65),
                                     (2, 512, 128, 384), (40, 64, 64, 64)])
def test_logbmm_double_backward_factored_on_the_matrix_cores(gpu, B, M, K, N):
    """genbmm_logbmm_bwdbwd_ws (eight matrix products on exp(a - max), exp(b - max), exp(max - out))
    against float64 second-order autograd, and against the exact vector-ALU passes of
    genbmm_logbmm_bwdbwd; full tiles, ragged extents in every position, each cotangent alone.
    Sums of up to 300 terms of magnitude |g u| <= ~20: absolute fp32 error well under 1e-4."""
    lib = _lib.load()
    assert lib.genbmm_logbmm_bwdbwd_ws_size(B, M, K, N) > B * M * N      # the factored form applies
    torch.manual_seed(M + N)
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    ua, ub = torch.randn(B, M, K), torch.randn(B, K, N)
    ad, bd, gd, uad, ubd = (t.to(gpu) for t in (a, b, g, ua, ub))
    out = genbmm.logbmm(ad, bd)
    pick = sorted({0, B // 2, B - 1})
    for u_a, u_b, ha, hb in ((uad, ubd, ua, ub), (uad, None, ua, None), (None, ubd, None, ub)):
        got = _bwdbwd_abi(gpu, ad, bd, out, gd, u_a, u_b, True)
        exact = _bwdbwd_abi(gpu, ad, bd, out, gd, u_a, u_b, False)
        for x, y in zip(got, exact):
            close(x, y, rtol=1e-4, atol=1e-4)
        want = oracle.logbmm_second_order64(a[pick], b[pick], g[pick], None if ha is None else ha[pick],
                                            None if hb is None else hb[pick])
        for x, y in zip(got, want):
            close(x[pick], y, rtol=1e-4, atol=1e-4)


def test_logbmm_double_backward_factored_guard(gpu):
    """Batch items with rows whose maxima sit on terms that never meet (the factors underflow
    against terms that matter), a -inf mask and a row at the floor: those items are redone by
    the exact passes, the others stay on the matrix cores; all agree with the exact passes."""
    torch.manual_seed(23)
    B, M, K, N = 6, 128, 96, 160
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    a[1, ::2, 0] += 200.0          # item 1: exp(a - rowmax) underflows for every k > 0 of those rows ...
    b[1, 0, :] -= 200.0            # ... while the true terms do not
    b[3, 5, :] = -float("inf")     # item 3: a masked k (stays factorable: exp -> 0)
    a[4, 7, :] = -1e9              # item 4: a row at the floor
    ua, ub = torch.randn(B, M, K), torch.randn(B, K, N)
    ad, bd, gd, uad, ubd = (t.to(gpu) for t in (a, b, g, ua, ub))
    gd[4, 7, :] = 0                # no gradient flows into the padding row
    out = genbmm.logbmm(ad, bd)
    got = _bwdbwd_abi(gpu, ad, bd, out, gd, uad, ubd, True)
    exact = _bwdbwd_abi(gpu, ad, bd, out, gd, uad, ubd, False)
    # (the weights of the row at the floor are a matter of rounding - a + b = out = -1e9 in float,
    # every weight 1, in the exact passes; the softmax of b's column in exact arithmetic and in the
    # factored form - so its own cells of grad_a and grad_g are left out; nothing flows out of it)
    for x, y, rowwise in zip(got, exact, (True, False, True)):
        x, y = x.clone(), y.clone()
        if rowwise:
            assert bool(torch.isfinite(x[4, 7]).all())
            x[4, 7], y[4, 7] = 0, 0
        fin = torch.isfinite(y)
        assert torch.equal(torch.isfinite(x), fin)
        close(x[fin], y[fin], rtol=1e-4, atol=1e-4)
    keep = [0, 1, 2, 3, 5]
    want = oracle.logbmm_second_order64(a[keep], b[keep], g[keep], ua[keep], ub[keep])
    for x, y in zip(got, want):
        close(x[keep], y, rtol=1e-4, atol=2e-4)


@pytest.mark.parametrize("B,M,K,N,flagged", [
    (40, 64, 64, 64, list(range(0, 40, 3)) + [39]),   # many flagged items, several to a group of workgroups
    (70, 128, 64, 64, [0, 63, 64, 69]),               # more than 64 items: two words of flags
    (2, 768, 64, 768, [1]),                           # an item of more blocks than the walking grid has workgroups
])
def test_logbmm_double_backward_flagged_items_walk(gpu, B, M, K, N, flagged):
    """The exact passes behind the factored form visit the flagged items only, a group of workgroups
    per item: every flagged item comes out as the exact passes alone give it (bit for bit), every
    other item within the factored form's tolerance."""
    torch.manual_seed(B + M)
    a, b = torch.randn(B, M, K, device=gpu), torch.randn(B, K, N, device=gpu)
    g, ua, ub = torch.randn(B, M, N, device=gpu), torch.randn(B, M, K, device=gpu), torch.randn(B, K, N, device=gpu)
    for i in flagged:              # rows whose maximum sits on a term that never meets a live one
        a[i, ::2, 0] += 200.0
        b[i, 0, :] -= 200.0
    out = genbmm.logbmm(a, b)
    got = _bwdbwd_abi(gpu, a, b, out, g, ua, ub, True)
    exact = _bwdbwd_abi(gpu, a, b, out, g, ua, ub, False)
    rest = [i for i in range(B) if i not in flagged]
    for x, y in zip(got, exact):
        assert torch.equal(x[flagged], y[flagged])
        close(x[rest], y[rest], rtol=1e-4, atol=2e-4)


def test_logbmm_double_backward_at_the_headline_shape(gpu):
    """(64, 512, 512, 512) through autograd with create_graph; three batch items against float64
    second-order autograd evaluated on the device."""
    torch.manual_seed(29)
    B, M, K, N = 64, 512, 512, 512
    ad, bd, gd = (torch.randn(B, M, K, device=gpu).requires_grad_(True), torch.randn(B, K, N, device=gpu).requires_grad_(True),
                  torch.randn(B, M, N, device=gpu).requires_grad_(True))
    ua = torch.randn(B, M, K, device=gpu)
    out = genbmm.logbmm(ad, bd)
    ga, gb = torch.autograd.grad(out, (ad, bd), gd, create_graph=True)
    got = torch.autograd.grad(ga, (ad, bd, gd), ua)                   # the reference's case: u_b absent
    for item in (0, 31, 63):
        sl = slice(item, item + 1)
        want = oracle.logbmm_second_order64(ad[sl], bd[sl], gd[sl], ua[sl], None)
        for x, y, what in zip(got, want, ("grad_a", "grad_b", "grad_g")):
            close_on_device(x[sl], y, "%s item %d" % (what, item), rtol=1e-4, atol=2e-4)
        del want


# ------------------------------------------------------------ max / prod-max
def grid(*shape):
    return torch.round(torch.randn(*shape) * 8) / 8


@pytest.mark.parametrize("B,M,K,N", [(4, 9, 17, 6), (3, 64, 64, 64), (2, 130, 70, 129), (5, 32, 32, 32),
                                     (2, 1, 1, 1), (2, 128, 200, 256), (16, 128, 48, 128)])
@pytest.mark.parametrize("prod", [False, True])
def test_max_forward_backward_bit_exact(gpu, B, M, K, N, prod):
    torch.manual_seed(M + K)
    if prod:
        a, b = 1 - torch.rand(B, M, K), 1 - torch.rand(B, K, N)
        a[:, :, ::3] = torch.round(a[:, :, ::3] * 4) / 4 + 0.25  # some exact product ties
        b[:, ::3, :] = torch.round(b[:, ::3, :] * 4) / 4 + 0.25
        op, orc = genbmm.prodmaxbmm, oracle.prodmaxbmm_broadcast
    else:
        a, b = grid(B, M, K), grid(B, K, N)
        op, orc = genbmm.maxbmm, oracle.maxbmm_broadcast
    g = grid(B, M, N).clamp(-4, 4)
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = op(ad, bd)
    wv, wi = orc(a, b)
    assert torch.equal(out.detach().cpu(), wv)
    sv, si = oracle.seq_maxbmm_fwd(a, b, prod)
    assert torch.equal(wv, sv) and torch.equal(wi.int(), si)
    ga, gb = torch.autograd.grad(out, (ad, bd), g.to(gpu))
    wa, wb = oracle.seq_argmax_bwd(a if prod else K, b, si, g, prod)
    assert torch.equal(ga.cpu(), wa), float((ga.cpu() - wa).abs().max())
    assert torch.equal(gb.cpu(), wb), float((gb.cpu() - wb).abs().max())


def _abi_max(gpu, a, b, prod, factors=None):
    lib = _lib.load()
    B, M, K = a.shape
    N = b.shape[2]
    out = torch.empty(B, M, N, device=gpu)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
    if prod:
        rc = lib.genbmm_prodmaxbmm_fwd(_lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(idx),
                                       _lib.ptr(factors), B, M, K, N, _lib.stream_of(a))
    else:
        rc = lib.genbmm_maxbmm_fwd(_lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(idx), B, M, K, N,
                                   _lib.stream_of(a))
    assert rc == 0
    return out, idx


@pytest.mark.parametrize("B,M,K,N", [(3, 70, 90, 50), (2, 64, 261, 130), (2, 130, 16, 64)])
def test_prodmax_factors_workspace(gpu, B, M, K, N):
    """The optional workspace of the prod-max forward holds a[m, idx] and b[idx, n]; the
    backward gives the same bits from it (a, b not passed) as from gathering a and b."""
    torch.manual_seed(N)
    a, b = grid(B, M, K), grid(B, K, N)
    a[:, ::5, ::3] *= 0
    g = grid(B, M, N).clamp(-4, 4)
    ad, bd, gd = a.to(gpu), b.to(gpu), g.to(gpu)
    fac = torch.full((2, B, M, N), float("nan"), device=gpu)
    out, idx = _abi_max(gpu, ad, bd, True, fac)
    out0, idx0 = _abi_max(gpu, ad, bd, True, None)
    sv, si = oracle.seq_maxbmm_fwd(a, b, True)
    assert torch.equal(out.cpu(), sv) and torch.equal(idx.cpu(), si)
    assert torch.equal(out0.cpu(), sv) and torch.equal(idx0.cpu(), si)
    li = si.long().clamp(min=0)
    want_a = torch.gather(a.unsqueeze(2).expand(B, M, N, K), 3, li.unsqueeze(-1)).squeeze(-1)
    want_b = torch.gather(b, 1, li)
    hit = si >= 0
    assert torch.equal(fac[0].cpu()[hit], want_a[hit]) and torch.equal(fac[1].cpu()[hit], want_b[hit])
    assert bool((fac[0].cpu()[~hit] == 0).all()) and bool((fac[1].cpu()[~hit] == 0).all())
    lib = _lib.load()
    res = []
    for use in (True, False):
        ga, gb = torch.full_like(ad, float("nan")), torch.full_like(bd, float("nan"))
        rc = lib.genbmm_prodmax_bwd(_lib.ptr(None if use else ad), _lib.ptr(None if use else bd), _lib.ptr(idx),
                                    _lib.ptr(fac if use else None), _lib.ptr(gd), _lib.ptr(ga), _lib.ptr(gb),
                                    B, M, K, N, _lib.stream_of(ad))
        assert rc == 0
        res.append((ga.cpu(), gb.cpu()))
    wa, wb = oracle.seq_argmax_bwd(a, b, si, g, True)
    for ga, gb in res:
        assert torch.equal(ga, wa) and torch.equal(gb, wb)
    # neither a/b nor the workspace: refused
    rc = lib.genbmm_prodmax_bwd(_lib.ptr(None), _lib.ptr(None), _lib.ptr(idx), _lib.ptr(None), _lib.ptr(gd),
                                _lib.ptr(ga.to(gpu)), _lib.ptr(gb.to(gpu)), B, M, K, N, _lib.stream_of(ad))
    assert rc != 0


@pytest.mark.parametrize("prod", [False, True])
def test_max_index_through_c_abi(gpu, prod):
    torch.manual_seed(3)
    a, b = grid(6, 70, 90), grid(6, 90, 50)
    if prod:
        a, b = a.abs() + 0.125, b.abs() + 0.125
    out, idx = _abi_max(gpu, a.to(gpu), b.to(gpu), prod)
    sv, si = oracle.seq_maxbmm_fwd(a, b, prod)
    assert torch.equal(out.cpu(), sv) and torch.equal(idx.cpu(), si)
    # floor: everything below -1e9 -> value -1e9, index -1 (matmul_cuda_kernel.cu:62-64)
    if not prod:
        lo = torch.full((1, 3, 4), -2e9)
        out, idx = _abi_max(gpu, lo.to(gpu), torch.zeros(1, 4, 2, device=gpu), False)
        assert bool((out == -1e9).all()) and bool((idx == -1).all())


@pytest.mark.parametrize("B,M,K,N", [(2, 70, 261, 65), (1, 40, 600, 130), (3, 33, 7, 20), (2, 64, 512, 128)])
@pytest.mark.parametrize("prod", [False, True])
def test_max_index_groups_and_special_values(gpu, prod, B, M, K, N):
    """The forward finds the index in two levels (group of consecutive k, then k inside
    the group, with the rows of b staged 256 at a time): K across several stages and
    not a multiple of the group, many ties, and NaN / infinite / signed-zero terms.
    Values are compared as bit patterns."""
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
    b[0, :, 0] = torch.where(torch.arange(K) % 3 == 0, 0.0, -0.0)
    out, idx = _abi_max(gpu, a.to(gpu), b.to(gpu), prod)
    sv, si = oracle.seq_maxbmm_fwd(a, b, prod)
    assert torch.equal(idx.cpu(), si)
    assert torch.equal(out.cpu().view(torch.int32), sv.view(torch.int32))
    assert int((si >= 0).sum()) > 0


def test_max_config_c3(gpu):
    """Benchmark configuration 2: (256,256,256) on the 1/8 grid (max) and Uniform(0,1] (prod-max).
    EVERY batch item: values and indices bit-exact against the broadcast closed form evaluated
    on the device in the operands' own precision (one rounding per term, as the reference;
    index = the lowest k that attains the maximum), max gradients bit-exact against the
    one-hot scatter (g on the 1/8 grid: sums exact in any order), prod-max gradients against
    the float64 scatter; a batch subset bit-exact against the sequential oracle (which also
    pins the order of the prod-max sums)."""
    torch.manual_seed(0)
    B = M = K = N = 256
    g = grid(B, M, N).clamp(-4, 4)
    gd = g.to(gpu)
    for prod in (False, True):
        if prod:
            a, b = 1 - torch.rand(B, M, K), 1 - torch.rand(B, K, N)
            op = genbmm.prodmaxbmm
        else:
            a, b = grid(B, M, K), grid(B, K, N)
            op = genbmm.maxbmm
        ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
        out = op(ad, bd)
        ga, gb = torch.autograd.grad(out, (ad, bd), gd)
        _, idx = _abi_max(gpu, ad.detach(), bd.detach(), prod)
        pick = [0, 101, 255]
        sv, si = oracle.seq_maxbmm_fwd(a[pick], b[pick], prod)
        assert torch.equal(out[pick].detach().cpu(), sv) and torch.equal(idx[pick].cpu(), si)
        wa, wb = oracle.seq_argmax_bwd(a[pick] if prod else K, b[pick], si, g[pick], prod)
        assert torch.equal(ga[pick].cpu(), wa) and torch.equal(gb[pick].cpu(), wb)
        # every item, on the device
        ks = torch.arange(K, device=gpu).view(1, 1, K, 1)
        ties = 0
        for i in range(0, B, 16):
            sl = slice(i, i + 16)
            x, y = ad[sl].detach().unsqueeze(-1), bd[sl].detach().unsqueeze(-3)
            s = x * y if prod else x + y                                          # (16, M, K, N)
            mv = s.max(-2).values
            hit = s == mv.unsqueeze(-2)
            first = torch.where(hit, ks, torch.full_like(ks, K)).min(-2).values
            assert torch.equal(out[sl].detach(), mv), i
            assert torch.equal(idx[sl].long(), first), i
            ties += int((hit.sum(-2) > 1).sum())
            li = first
            if prod:   # float64 scatter of b[idx, n] * g (resp. a[m, idx] * g); the order of the fp32 sums: subset above
                wa64 = torch.zeros(16, M, K, device=gpu, dtype=torch.float64)
                wb64 = torch.zeros(16, K, N, device=gpu, dtype=torch.float64)
                bsel = torch.gather(bd[sl].detach(), 1, li).double()
                asel = torch.gather(ad[sl].detach().unsqueeze(2).expand(16, M, N, K), 3, li.unsqueeze(-1)).squeeze(-1).double()
                wa64.scatter_add_(2, li, bsel * gd[sl].double())
                wb64.scatter_add_(1, li, asel * gd[sl].double())
                assert torch.allclose(ga[sl].double(), wa64, rtol=1e-5, atol=1e-5), i
                assert torch.allclose(gb[sl].double(), wb64, rtol=1e-5, atol=1e-5), i
            else:
                wa32 = torch.zeros(16, M, K, device=gpu).scatter_add_(2, li, gd[sl])
                wb32 = torch.zeros(16, K, N, device=gpu).scatter_add_(1, li, gd[sl])
                assert torch.equal(ga[sl], wa32) and torch.equal(gb[sl], wb32), i
            del s, hit, first, mv
        if not prod:
            assert ties > 100 * B   # ties are present in this configuration and resolve to the lowest k


# -------------------------------------------------------------------- sample
@pytest.mark.parametrize("use_stats", [True, False])
@pytest.mark.parametrize("B,M,K,N", [(6, 20, 37, 24), (3, 130, 64, 132), (2, 64, 100, 128),
                                     # shapes whose forward leaves the factors: two-level sweep (groups of 8
                                     # terms; K not a multiple of 8, K across several staged chunks / folds)
                                     (2, 128, 96, 160), (2, 200, 100, 260), (2, 256, 520, 128), (1, 97, 1030, 96)])
def test_sample_index_brackets_cdf(gpu, use_stats, B, M, K, N):
    torch.manual_seed(11)
    a, b = 2 * torch.randn(B, M, K), 2 * torch.randn(B, K, N)
    a[0, ::2, 0] += 150.0      # batch item 0: the factored walk is not exact -> exact walk
    b[0, 0, :] -= 150.0
    seed, offset = 1234, 5
    lib = _lib.load()
    ad, bd = a.to(gpu), b.to(gpu)
    out = torch.empty(B, M, N, device=gpu)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
    stats = torch.empty(lib.genbmm_samplebmm_stats_size(B, M, K, N), device=gpu) if use_stats else None
    rc = lib.genbmm_samplebmm_fwd(_lib.ptr(ad), _lib.ptr(bd), _lib.ptr(out), _lib.ptr(idx), _lib.ptr(stats),
                                  seed, offset, B, M, K, N, _lib.stream_of(ad))
    assert rc == 0
    close(out, lse64(a, b))
    u = oracle.philox_uniform(0, B * M * N, seed, offset).view(B, M, N)
    cdf = oracle.sample_cdf64(a, b)                                   # (B,M,K,N)
    got = idx.cpu().long()
    want = oracle.sample_index_from_cdf(cdf, u).long()
    assert float((got != want).float().mean()) < 2e-3
    # every index brackets its uniform up to fp32 rounding of the CDF
    hi = torch.gather(cdf, 2, got.unsqueeze(2)).squeeze(2)
    lo = torch.where(got > 0, torch.gather(cdf, 2, (got - 1).clamp(min=0).unsqueeze(2)).squeeze(2),
                     torch.zeros_like(hi))
    tol = 2e-5
    ok = (lo - tol <= u.double()) & (u.double() <= hi + tol)
    assert bool(ok.all())
    # same stream -> same draw; other offset -> different draw
    idx2 = torch.empty_like(idx)
    lib.genbmm_samplebmm_fwd(_lib.ptr(ad), _lib.ptr(bd), _lib.ptr(out), _lib.ptr(idx2), _lib.ptr(stats),
                             seed, offset, B, M, K, N, _lib.stream_of(ad))
    assert torch.equal(idx, idx2)
    lib.genbmm_samplebmm_fwd(_lib.ptr(ad), _lib.ptr(bd), _lib.ptr(out), _lib.ptr(idx2), _lib.ptr(stats),
                             seed, offset + 1, B, M, K, N, _lib.stream_of(ad))
    assert not torch.equal(idx, idx2)


@pytest.mark.parametrize("B,M,K,N", [(2, 40, 4096, 30), (1, 16, 6000, 16), (2, 100, 2101, 97), (1, 7, 8192, 5)])
def test_sample_on_long_reductions_with_few_tiles(gpu, B, M, K, N):
    """samplebmm on a problem whose forward cuts the reduction axis into pieces: the draw picks the
    piece in which the prefix of the pieces' sums passes the cell's target and walks that piece.
    out against float64; every index brackets its Philox uniform in the float64 CDF (tolerance:
    the rounding of an fp32 sum of K terms); batch item 0 holds rows that defeat the factoring
    (flagged tiles walk the reference's own way); same stream, same draw; float16 operands too."""
    lib = _lib.load()
    assert lib.genbmm_logbmm_fwd_pieces(B, M, K, N) > 1
    torch.manual_seed(K + N)
    a, b = 2 * torch.randn(B, M, K), 2 * torch.randn(B, K, N)
    a[0, ::2, 0] += 150.0
    b[0, 0, :] -= 150.0
    seed, offset = 4321, 2
    u = oracle.philox_uniform(0, B * M * N, seed, offset).view(B, M, N).double()
    tol = max(2e-5, K * 2.0 ** -24)
    for dt, suffix in ((torch.float32, ""), (torch.float16, "_f16")):
        ad, bd = a.to(gpu).to(dt), b.to(gpu).to(dt)
        a32, b32 = ad.float().cpu(), bd.float().cpu()
        out = torch.empty(B, M, N, device=gpu, dtype=dt)
        idx = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
        stats = torch.empty(lib.genbmm_samplebmm_stats_size(B, M, K, N), device=gpu)
        fn = getattr(lib, "genbmm_samplebmm_fwd" + suffix)
        assert fn(_lib.ptr(ad), _lib.ptr(bd), _lib.ptr(out), _lib.ptr(idx), _lib.ptr(stats), seed, offset, B, M, K, N,
                  _lib.stream_of(ad)) == 0
        want = lse64(a32, b32)
        if dt == torch.float32:
            close(out, want)
        else:
            assert bool(((out.double().cpu() - want).abs() <= 2.0 ** -11 * want.abs() + 1e-5 * want.abs() + 1e-6).all())
        cdf = oracle.sample_cdf64(a32, b32)                               # (B,M,K,N)
        got = idx.cpu().long()
        assert int(got.min()) >= 0 and int(got.max()) < K
        hi = torch.gather(cdf, 2, got.unsqueeze(2)).squeeze(2)
        lo = torch.where(got > 0, torch.gather(cdf, 2, (got - 1).clamp(min=0).unsqueeze(2)).squeeze(2),
                         torch.zeros_like(hi))
        ok = (lo - tol <= u) & (u <= hi + tol)
        assert bool(ok.all()), (str(dt), float((~ok).float().mean()))
        assert float((got != oracle.sample_index_from_cdf(cdf, u).long()).float().mean()) < 5e-3
        idx2 = torch.empty_like(idx)
        fn(_lib.ptr(ad), _lib.ptr(bd), _lib.ptr(out), _lib.ptr(idx2), _lib.ptr(stats), seed, offset, B, M, K, N,
           _lib.stream_of(ad))
        assert torch.equal(idx, idx2)
    # through the public function: the one-hot gradient of the drawn term
    ar = a.to(gpu).requires_grad_(True)
    o = genbmm.samplebmm(ar, b.to(gpu), (seed, offset))
    (ga,) = torch.autograd.grad(o.sum(), ar)
    assert float(ga.sum()) == pytest.approx(B * M * N, rel=1e-3)


def test_sample_config_c4_chi_square(gpu):
    """Benchmark configuration 3: Normal(0,2) (64,512,512) potentials, Philox seed 1234; 10^4
    draws per cell of the (4,16,16) slice; per-cell chi-square against the float64
    softmax, categories with expected count < 5 pooled, bound = the 1-1e-6 quantile."""
    from scipy.stats import chi2 as chi2_dist

    torch.manual_seed(0)
    a, b = 2 * torch.randn(64, 512, 512), 2 * torch.randn(64, 512, 512)
    sa, sb = a[:4, :16, :].contiguous(), b[:4, :, :16].contiguous()
    draws = 10000
    A = sa.repeat(draws, 1, 1).to(gpu).requires_grad_(True)           # (40000,16,512)
    Bm = sb.repeat(draws, 1, 1).to(gpu)
    out = genbmm.samplebmm(A, Bm, (1234, 0))
    # the gradient is the one-hot sample: histogram it through grad_a-like counts
    lib = _lib.load()
    idx = torch.empty(A.shape[0], 16, 16, dtype=torch.int32, device=gpu)
    o2 = torch.empty_like(out)
    st = torch.empty(lib.genbmm_samplebmm_stats_size(A.shape[0], 16, 512, 16), device=gpu)
    lib.genbmm_samplebmm_fwd(_lib.ptr(A), _lib.ptr(Bm), _lib.ptr(o2), _lib.ptr(idx), _lib.ptr(st), 1234, 0,
                             A.shape[0], 16, 512, 16, _lib.stream_of(A))
    assert torch.equal(o2, out.detach())
    (gA,) = torch.autograd.grad(out.sum(), (A,))                      # one-hot rows summed over n
    onehot = torch.zeros(A.shape[0], 16, 512, device=gpu)
    onehot.scatter_add_(2, idx.long(), torch.ones_like(idx, dtype=torch.float32))
    assert torch.equal(gA, onehot)
    counts = torch.zeros(4, 16, 16, 512, dtype=torch.float64)
    iv = idx.view(draws, 4, 16, 16).cpu().long()
    counts.scatter_add_(3, iv.permute(1, 2, 3, 0), torch.ones(4, 16, 16, draws, dtype=torch.float64))
    p = torch.softmax(sa.double().unsqueeze(-1) + sb.double().unsqueeze(-3), -2).permute(0, 1, 3, 2)
    expc = p * draws                                                  # (4,16,16,512)
    worst = 0.0
    for cell in range(4 * 16 * 16):
        e, c = expc.reshape(-1, 512)[cell], counts.reshape(-1, 512)[cell]
        keep = e >= 5
        stat = float((((c - e) ** 2) / e)[keep].sum())
        dof = int(keep.sum())
        if (~keep).any():
            ep, cp = float(e[~keep].sum()), float(c[~keep].sum())
            if ep >= 1:
                stat += (cp - ep) ** 2 / ep
                dof += 1
        dof = max(dof - 1, 1)
        bound = chi2_dist.ppf(1 - 1e-6, dof)
        worst = max(worst, stat / bound)
        assert stat < bound, (cell, stat, bound, dof)
    assert worst > 0


def test_sample_config_c4_at_full_size(gpu):
    """Benchmark configuration 3 at its own size, through the C ABI: a, b = 2 * randn
    (64, 512, 512) from seed 0, Philox seed 1234 - the shape whose sweep runs on the
    matrix cores in 128 x 128 tiles behind a 256 x 128 forward.
    out against the float64 log-sum-exp and every index against the float64 CDF of its
    cell on a batch subset; over everything: 0 <= idx < K, the picked term carries mass,
    and the one-hot gradients add up to g along k (exactly, g on the 1/8 grid).  Then the
    chi-square of the slice test above, with the 10^4 draws per cell taken from 10^4
    full-size calls (distinct Philox offsets) instead of from a tiled copy of the slice."""
    from scipy.stats import chi2 as chi2_dist

    torch.manual_seed(0)
    B, M, K, N = 64, 512, 512, 512
    a, b = 2 * torch.randn(B, M, K), 2 * torch.randn(B, K, N)
    lib = _lib.load()
    ad, bd = a.to(gpu), b.to(gpu)
    out = torch.empty(B, M, N, device=gpu)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
    stats = torch.empty(lib.genbmm_samplebmm_stats_size(B, M, K, N), device=gpu)
    p, s = _lib.ptr, _lib.stream_of(ad)

    def draw(offset):
        assert lib.genbmm_samplebmm_fwd(p(ad), p(bd), p(out), p(idx), p(stats), 1234, offset, B, M, K, N, s) == 0

    draw(0)
    u = oracle.philox_uniform(0, B * M * N, 1234, 0).view(B, M, N)
    for item in (0, 37, 63):
        close(out[item:item + 1], lse64(a[item:item + 1], b[item:item + 1]))
        # the oracle's float64 CDF, evaluated on the device (1 GiB per batch item)
        cdf = oracle.sample_cdf64(ad[item:item + 1], bd[item:item + 1])
        got = idx[item:item + 1].long()
        hi = torch.gather(cdf, 2, got.unsqueeze(2)).squeeze(2)
        lo = torch.where(got > 0, torch.gather(cdf, 2, (got - 1).clamp(min=0).unsqueeze(2)).squeeze(2),
                         torch.zeros_like(hi))
        ui = u[item:item + 1].to(gpu).double()
        ok = (lo - 2e-5 <= ui) & (ui <= hi + 2e-5)
        assert bool(ok.all()), (item, float((~ok).float().mean()))
        want = oracle.sample_index_from_cdf(cdf, ui).long()
        assert float((got != want).float().mean()) < 2e-3
        del cdf, want
    il = idx.long()
    assert int(il.min()) >= 0 and int(il.max()) < K
    picked = torch.gather(ad, 2, il) + torch.gather(bd, 1, il)       # a[m, idx] + b[idx, n]
    assert bool((picked - out > -40.0).all())                         # a term of visible mass
    g = (torch.round(torch.randn(B, M, N) * 8) / 8).clamp(-4, 4).to(gpu)
    ga, gb = torch.empty_like(ad), torch.empty_like(bd)
    assert lib.genbmm_argmax_bwd(p(idx), p(g), p(ga), p(gb), B, M, K, N, s) == 0
    assert torch.equal(ga.sum(-1), g.sum(-1)) and torch.equal(gb.sum(-2), g.sum(-2))
    onehot = torch.zeros(M, K, device=gpu).scatter_add_(1, il[5], g[5])
    assert torch.equal(ga[5], onehot)

    # chi-square on the (4,16,16) slice from full-size draws
    draws = 10000
    counts = torch.zeros(4 * 16 * 16, K, device=gpu)
    cells = torch.arange(4 * 16 * 16, device=gpu)
    one = torch.ones(4 * 16 * 16, device=gpu)
    for d in range(draws):
        draw(4 * d + 4)
        counts.index_put_((cells, idx[:4, :16, :16].reshape(-1).long()), one, accumulate=True)
    counts = counts.cpu().double().view(4, 16, 16, K)
    pr = torch.softmax(a[:4, :16, :].double().unsqueeze(-1) + b[:4, :, :16].double().unsqueeze(-3), -2)
    expc = pr.permute(0, 1, 3, 2) * draws                             # (4,16,16,K)
    for cell in range(4 * 16 * 16):
        e, c = expc.reshape(-1, K)[cell], counts.reshape(-1, K)[cell]
        keep = e >= 5
        stat = float((((c - e) ** 2) / e)[keep].sum())
        dof = int(keep.sum())
        if (~keep).any():
            ep, cp = float(e[~keep].sum()), float(c[~keep].sum())
            if ep >= 1:
                stat += (cp - ep) ** 2 / ep
                dof += 1
        dof = max(dof - 1, 1)
        assert stat < chi2_dist.ppf(1 - 1e-6, dof), (cell, stat, dof)


def test_sample_distribution_on_the_matrix_core_sweep(gpu):
    """A shape whose sweep runs on the matrix cores (slabs of 16 terms + resolve): 1500
    draws per cell with distinct Philox offsets; the empirical CDF of every cell stays
    within the Kolmogorov-Smirnov band of the float64 softmax CDF (1e-9 quantile:
    sqrt(ln(2e9) / 3000) = 0.0845)."""
    torch.manual_seed(21)
    B, M, K, N, draws = 2, 128, 80, 128, 1500
    a, b = 2 * torch.randn(B, M, K), 2 * torch.randn(B, K, N)
    lib = _lib.load()
    ad, bd = a.to(gpu), b.to(gpu)
    out = torch.empty(B, M, N, device=gpu)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
    stats = torch.empty(lib.genbmm_samplebmm_stats_size(B, M, K, N), device=gpu)
    counts = torch.zeros(B * M * N, K, device=gpu)
    cells = torch.arange(B * M * N, device=gpu)
    for d in range(draws):
        rc = lib.genbmm_samplebmm_fwd(_lib.ptr(ad), _lib.ptr(bd), _lib.ptr(out), _lib.ptr(idx), _lib.ptr(stats),
                                      99, 7 * d, B, M, K, N, _lib.stream_of(ad))
        assert rc == 0
        counts[cells, idx.view(-1).long()] += 1
    close(out, lse64(a, b))
    emp = (counts.cumsum(1) / draws).cpu().double().view(B, M, N, K).permute(0, 1, 3, 2)   # (B,M,K,N)
    cdf = oracle.sample_cdf64(a, b)
    assert float((emp - cdf).abs().max()) < 0.0845
    # and not degenerate: the draws differ from offset to offset
    assert float((counts.max(1).values < draws).float().mean()) > 0.9


def test_sample_public_api_follows_torch_seed(gpu):
    a, b = torch.randn(3, 8, 16, device=gpu, requires_grad=True), torch.randn(3, 16, 8, device=gpu)
    torch.manual_seed(5)
    g1 = torch.autograd.grad(genbmm.samplebmm(a, b).sum(), a)[0]
    g2 = torch.autograd.grad(genbmm.samplebmm(a, b).sum(), a)[0]
    torch.manual_seed(5)
    g3 = torch.autograd.grad(genbmm.samplebmm(a, b).sum(), a)[0]
    assert torch.equal(g1, g3) and not torch.equal(g1, g2)
    assert torch.equal(g1.sum(-1), torch.full((3, 8), 8.0, device=gpu))  # one sample per (m,n)


# ------------------------------------------------------------ error handling
def test_errors(gpu):
    a, b = torch.randn(2, 3, 4), torch.randn(2, 4, 5)
    for op in (genbmm.logbmm, genbmm.maxbmm, genbmm.samplebmm, genbmm.prodmaxbmm):
        with pytest.raises(RuntimeError, match="CUDA tensor"):
            op(a, b)                                                   # matmul_cuda.cpp:65
        with pytest.raises(RuntimeError, match="shape mismatch"):
            op(a.to(gpu), torch.randn(2, 3, 5, device=gpu))
        with pytest.raises(RuntimeError, match="same dtype"):
            op(a.to(gpu).double(), b.to(gpu))
        with pytest.raises(RuntimeError, match="not supported"):
            op(a.to(gpu).long(), b.to(gpu).long())
    # the autograd Functions themselves keep the reference's contract (matmul_cuda.cpp:66)
    with pytest.raises(RuntimeError, match="contiguous"):
        genmul.LogMatMul.apply(a.to(gpu).transpose(1, 2).contiguous().transpose(1, 2), b.to(gpu))
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    ad = a.to(gpu)
    assert lib.genbmm_logbmm_fwd_path(_lib.ptr(ad), _lib.ptr(ad), _lib.ptr(ad), null, 1, 1, 1, 1, 7, null) == -3
    assert lib.genbmm_logbmm_fwd(null, _lib.ptr(ad), _lib.ptr(ad), null, 1, 1, 1, 1, null) == -1
    assert lib.genbmm_logbmm_fwd(_lib.ptr(ad), _lib.ptr(ad), _lib.ptr(ad), null, 1, -1, 1, 1, null) == -2
    assert lib.genbmm_banded_fwd(_lib.ptr(ad), 0, 0, _lib.ptr(ad), 0, 0, _lib.ptr(ad), null, null, 1, 1, 2, null) == -3
    assert lib.genbmm_banded_fwd(_lib.ptr(ad), -1, 0, _lib.ptr(ad), 0, 0, _lib.ptr(ad), null, null, 1, 1, 0, null) == -4
    assert b"NULL" in lib.genbmm_error_string(-1)


def test_empty_and_half(gpu):
    for shape in [(0, 3, 4, 5), (2, 0, 4, 5), (2, 3, 4, 0)]:
        B, M, K, N = shape
        out = genbmm.logbmm(torch.randn(B, M, K, device=gpu), torch.randn(B, K, N, device=gpu))
        assert out.shape == (B, M, N)
    out = genbmm.logbmm(torch.randn(2, 3, 0, device=gpu), torch.randn(2, 0, 5, device=gpu))
    assert bool(torch.isinf(out).all())                              # empty sum: log(0) - 1e9
    a, b = torch.randn(2, 9, 12, device=gpu).half(), torch.randn(2, 12, 7, device=gpu).half()
    out = genbmm.logbmm(a.requires_grad_(True), b)
    assert out.dtype == torch.float16
    close(out.float(), lse64(a.float().cpu(), b.float().cpu()), rtol=2e-3, atol=2e-3)
    (ga,) = torch.autograd.grad(out.sum(), a)
    assert ga.dtype == torch.float16


def test_views_and_batch_dimensions(gpu):
    """Operands that are views (transposed, strided) are made contiguous, and any number
    of leading batch dimensions - equal or broadcastable - is accepted; gradients arrive
    in the callers' own tensors.  (The reference takes 3-D contiguous tensors only.)"""
    torch.manual_seed(11)
    at, b = torch.randn(3, 9, 14), torch.randn(3, 9, 6)       # a is given as the transpose of `at`
    g = torch.randn(3, 14, 6)
    want, wa, wb = oracle.logbmm_grads64(at.transpose(1, 2).contiguous(), b, g)
    atd, bd = at.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = genbmm.logbmm(atd.transpose(1, 2), bd)
    ga, gb = torch.autograd.grad(out, (atd, bd), g.to(gpu))
    close(out, want)
    close(ga, wa.transpose(1, 2))
    close(gb, wb)
    grid8 = lambda *s: torch.round(torch.randn(*s) * 8) / 8
    a5, b5 = grid8(2, 3, 4, 7, 5), grid8(3, 1, 5, 8)          # batch (2, 3, 4) against (3, 1): broadcast
    for op, ref in ((genbmm.maxbmm, lambda x, y: (x.unsqueeze(-1) + y.unsqueeze(-3)).amax(-2)),
                    (genbmm.prodmaxbmm, lambda x, y: (x.unsqueeze(-1) * y.unsqueeze(-3)).amax(-2))):
        x, y = a5.to(gpu).requires_grad_(True), b5.to(gpu).requires_grad_(True)
        got = op(x, y)
        assert got.shape == (2, 3, 4, 7, 8)
        assert torch.equal(got.cpu(), ref(a5, b5.expand(2, 3, 4, 5, 8)))
        gx, gy = torch.autograd.grad(got.sum(), (x, y))
        assert gx.shape == a5.shape and gy.shape == b5.shape
    s5 = genbmm.samplebmm(a5.to(gpu), b5.to(gpu), (7, 0))
    close(s5, lse64(a5.reshape(-1, 7, 5), b5.expand(2, 3, 4, 5, 8).reshape(-1, 5, 8)).reshape(2, 3, 4, 7, 8))
    a2, b2 = torch.randn(6, 5), torch.randn(5, 4)              # plain matrices
    close(genbmm.logbmm(a2.to(gpu), b2.to(gpu)), lse64(a2[None], b2[None])[0])


@pytest.mark.parametrize("B,M,K,N", [(2, 40, 4096, 30), (1, 7, 8192, 5), (1, 100, 4608, 96), (1, 16, 6000, 16)])
def test_long_reductions_with_few_tiles_are_split(gpu, B, M, K, N):
    """logbmm cuts a long reduction axis of a problem with few output tiles into batch items of
    its own and joins them by a logsumexp (host layer): same values, first and second
    derivatives as the float64 closed form.  (6000 = 2^4 * 3 * 5^3: the cut takes a divisor.)"""
    assert genmul._reduction_splits(B, M, K, N) > 1
    assert genmul._reduction_splits(64, 512, 512, 512) == 1 and genmul._reduction_splits(512, 128, 128, 128) == 1
    torch.manual_seed(K + M)
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    want, wa, wb = oracle.logbmm_grads64(a, b, g)
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = genbmm.logbmm(ad, bd)
    close(out, want)
    ga, gb = torch.autograd.grad(out, (ad, bd), g.to(gpu), create_graph=True)
    close(ga, wa)
    close(gb, wb)
    if B * M * K * N <= 3_000_000:
        u = torch.randn(B, M, K)
        w2 = oracle.logbmm_second_order64(a, b, g, u, None)
        da, db = torch.autograd.grad((ga * u.to(gpu)).sum(), (ad, bd))
        close(da, w2[0], rtol=1e-4, atol=1e-5)
        close(db, w2[1], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("B,M,K,N", [(16, 96, 4096, 96), (1, 16, 65536, 16), (60, 7, 4100, 7), (3, 130, 2101, 97),
                                     (2, 300, 5000, 200), (1, 64, 2048, 64)])
@pytest.mark.parametrize("prod", [False, True])
def test_library_cuts_long_max_reductions_into_pieces(gpu, prod, B, M, K, N):
    """genbmm_maxbmm_fwd / genbmm_prodmaxbmm_fwd cut the reduction axis of a problem with few
    output tiles into pieces whose maxima and lowest indices meet by integer atomics: values (as
    bit patterns), indices and the product semiring's factors equal to the sequential oracle's,
    with ties inside and across pieces, NaN / infinite / signed-zero terms, a row below the -1e9
    floor and a row of NaN; twice in a row into the same buffers; through autograd as well."""
    lib = _lib.load()
    assert lib.genbmm_maxbmm_fwd_pieces(B, M, K, N) > 1
    assert lib.genbmm_maxbmm_fwd_pieces(256, 256, 256, 256) == 1 and lib.genbmm_maxbmm_fwd_pieces(1, 16, 2000, 16) == 1
    assert lib.genbmm_maxbmm_fwd_pieces(4, 512, 8192, 512) == 1
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
    b[0, :, 0] = torch.where(torch.arange(K) % 3 == 0, 0.0, -0.0)
    a[-1, M - 1, :] = float("nan")    # no term at all: value -1e9, index -1
    if not prod:
        a[-1, 1 % M, :] = -3e9        # every term below the floor
    ad, bd = a.to(gpu), b.to(gpu)
    sv, si = oracle.seq_maxbmm_fwd(a, b, prod)
    fac = torch.full((2, B, M, N), float("nan"), device=gpu) if prod else None
    for _ in range(2):
        out, idx = _abi_max(gpu, ad, bd, prod, fac)
        assert torch.equal(idx.cpu(), si)
        assert torch.equal(out.cpu().view(torch.int32), sv.view(torch.int32))
    assert bool((si[-1, M - 1] == -1).all()) and int((si >= 0).sum()) > 0
    if prod:
        k = si.long().clamp(min=0)
        fa = torch.gather(a, 2, k)                                      # a[m, idx]
        fb = torch.gather(b, 1, k)                                      # b[idx, n]
        live = si >= 0
        assert torch.equal(fac[0].cpu()[live], fa[live]) and torch.equal(fac[1].cpu()[live], fb[live])
        assert bool((fac[0].cpu()[~live] == 0).all()) and bool((fac[1].cpu()[~live] == 0).all())
    # the public function leaves the cut to the library and its gradient is the one-hot scatter
    op = genbmm.prodmaxbmm if prod else genbmm.maxbmm
    a2, b2 = a.nan_to_num(nan=-1.0, posinf=3.0, neginf=-3.0), b.nan_to_num(nan=-1.0, posinf=3.0, neginf=-3.0)
    ar, br = a2.to(gpu).requires_grad_(True), b2.to(gpu).requires_grad_(True)
    o = op(ar, br)
    sv2, si2 = oracle.seq_maxbmm_fwd(a2, b2, prod)
    assert torch.equal(o.detach().cpu().view(torch.int32), sv2.view(torch.int32))
    g = grid(B, M, N).clamp(-4, 4)
    ga, gb = torch.autograd.grad(o, (ar, br), g.to(gpu))
    wa, wb = oracle.seq_argmax_bwd(a2 if prod else K, b2, si2, g, prod)
    assert torch.equal(ga.cpu(), wa) and torch.equal(gb.cpu(), wb)


@pytest.mark.parametrize("B,M,K,N", [(16, 96, 4096, 96), (1, 16, 65536, 16), (64, 7, 4100, 7), (3, 130, 2101, 97),
                                     (2, 300, 5000, 200), (1, 128, 2048, 128), (100, 120, 2300, 127)])
def test_library_cuts_long_reductions_into_pieces(gpu, B, M, K, N):
    """genbmm_logbmm_fwd cuts the reduction axis of a problem with few output tiles into pieces,
    one workgroup each, and joins their sums before the guard and the logarithm: values and both
    gradients (the ordinary backward on the forward's workspace) against float64; items whose
    tiles must take the exact routine (a factor that underflows against live terms), a row at the
    floor, a masked reduction step and a masked row; the workspace is larger by the pieces' sums;
    float16 / bfloat16 tensors on the same kernels; the entry point without allocation never cuts."""
    lib = _lib.load()
    pieces = lib.genbmm_logbmm_fwd_pieces(B, M, K, N)
    assert pieces > 1
    assert lib.genbmm_logbmm_fwd_pieces(64, 512, 512, 512) == 1 and lib.genbmm_logbmm_fwd_pieces(512, 128, 128, 128) == 1
    assert lib.genbmm_logbmm_fwd_pieces(1, 512, 8192, 4096) == 1 and lib.genbmm_logbmm_fwd_pieces(16, 64, 64, 64) == 1
    size = lib.genbmm_logbmm_stats_size(B, M, K, N)
    assert size >= pieces * B * M * N + B * (M + N)
    torch.manual_seed(K + M)
    a, b, g = torch.randn(B, M, K), torch.randn(B, K, N), torch.randn(B, M, N)
    a[0, ::2, 0] += 200.0           # the other terms' factors underflow: exact routine
    b[0, 0, :] -= 200.0
    a[B - 1, M - 1, :] = -1e9      # a row at the floor
    g[B - 1, M - 1, :] = 0.0
    b[B // 2, K - 3, :] = -float("inf")
    b[B // 2, :, N - 1] = -float("inf")   # a masked column: out = -inf
    ad, bd, gd = a.to(gpu), b.to(gpu), g.to(gpu)
    P, s = _lib.ptr, _lib.stream_of(ad)
    out, st = torch.empty(B, M, N, device=gpu), torch.empty(size, device=gpu)
    ga, gb = torch.empty_like(ad), torch.empty_like(bd)
    assert lib.genbmm_logbmm_fwd(P(ad), P(bd), P(out), P(st), B, M, K, N, s) == 0
    assert lib.genbmm_logbmm_bwd(P(ad), P(bd), P(out), P(gd), P(st), P(ga), P(gb), B, M, K, N, s) == 0
    torch.cuda.synchronize()
    want, wa, wb = oracle.logbmm_grads64(a, b, g)
    col = torch.ones(B, 1, N, dtype=torch.bool)
    col[B // 2, 0, N - 1] = False   # the masked column: -inf in out, nothing to compare in the gradients
    rows = torch.ones(B, M, 1, dtype=torch.bool)
    rows[B - 1, M - 1, 0] = False   # the floor row's own cells: rounding artefacts of 1e9
    assert bool(torch.isneginf(out[B // 2, :, N - 1]).all())
    keep = (col & rows).expand(B, M, N)
    close(out.cpu()[keep], want[keep])
    close(torch.where(rows.expand(B, M, K), ga.cpu(), torch.zeros(())), torch.where(rows.expand(B, M, K), wa, torch.zeros(())))
    close(torch.where(col.expand(B, K, N), gb.cpu(), torch.zeros(())), torch.where(col.expand(B, K, N), wb, torch.zeros(())))
    # the public function takes the same route (and its second derivative the library's)
    ar, br = ad.clone().requires_grad_(True), bd.clone().requires_grad_(True)
    o2 = genbmm.logbmm(ar, br)
    assert torch.equal(o2.detach(), out)
    # the entry point without allocation: no room for the pieces' sums, the unsplit kernels
    if lib.genbmm_logbmm_stats_size_path(B, M, K, N, genmul.PATH_MFMA32) <= lib.genbmm_logbmm_static_limit():
        o3 = torch.empty_like(out)
        assert lib.genbmm_logbmm_fwd_static(P(ad), P(bd), P(o3), B, M, K, N, s) == 0
        torch.cuda.synchronize()
        close(o3.cpu()[keep], want[keep])
    for dt, sfx, eps in ((torch.float16, "_f16", 2.0 ** -11), (torch.bfloat16, "_bf16", 2.0 ** -8)):
        ah, bh = ad.to(dt), bd.to(dt)
        oh = torch.empty(B, M, N, device=gpu, dtype=dt)
        assert getattr(lib, "genbmm_logbmm_fwd" + sfx)(P(ah), P(bh), P(oh), P(st), B, M, K, N, s) == 0
        o32 = torch.empty(B, M, N, device=gpu)
        a32, b32 = ah.float(), bh.float()
        assert lib.genbmm_logbmm_fwd(P(a32), P(b32), P(o32), P(st), B, M, K, N, s) == 0
        torch.cuda.synchronize()
        assert torch.equal(oh, o32.to(dt))


@pytest.mark.parametrize("B,M,K,N", [(2, 40, 4096, 30), (1, 7, 8192, 5), (1, 100, 4608, 96), (1, 16, 6000, 16)])
@pytest.mark.parametrize("prod", [False, True])
def test_long_reductions_of_the_max_products_are_split(gpu, prod, B, M, K, N):
    """maxbmm / prodmaxbmm cut a long reduction over few output tiles into batch items of its own
    and join the pieces' maxima (host layer): values, indices into the whole of K (ties to the
    lowest k, also across pieces) and gradients equal the sequential oracle's bit for bit."""
    assert genmul._reduction_splits(B, M, K, N) > 1
    torch.manual_seed(K + N)
    if prod:
        a, b = 1 - torch.rand(B, M, K), 1 - torch.rand(B, K, N)
    else:
        a, b = grid(B, M, K), grid(B, K, N)      # multiples of 1/8: many ties, within and across pieces
    g = grid(B, M, N).clamp(-4, 4)
    sv, si = oracle.seq_maxbmm_fwd(a, b, prod)
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = (genbmm.prodmaxbmm if prod else genbmm.maxbmm)(ad, bd)
    assert torch.equal(out.detach().cpu(), sv)
    ga, gb = torch.autograd.grad(out, (ad, bd), g.to(gpu))
    wa, wb = oracle.seq_argmax_bwd(a if prod else K, b, si, g, prod)
    assert torch.equal(ga.cpu(), wa) and torch.equal(gb.cpu(), wb)
    # half tensors: the float function on the widened tensors, rounded once
    ah, bh = a.half().to(gpu), b.half().to(gpu)
    oh = (genbmm.prodmaxbmm if prod else genbmm.maxbmm)(ah, bh)
    of = (genbmm.prodmaxbmm if prod else genbmm.maxbmm)(ah.float(), bh.float())
    assert oh.dtype == torch.float16 and torch.equal(oh, of.half())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_long_reductions_split_with_half_tensors(gpu, dtype):
    """The split of a long reduction on float16 / bfloat16 operands keeps the half contract: what
    the float function returns on the widened tensors, rounded once (pieces are formed and joined
    in float32) - forward and gradients, bit for bit."""
    B, M, K, N = 2, 40, 4096, 30
    assert genmul._reduction_splits(B, M, K, N) > 1
    torch.manual_seed(3)
    a, b, g = torch.randn(B, M, K).to(dtype), torch.randn(B, K, N).to(dtype), torch.randn(B, M, N).to(dtype)
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    out = genbmm.logbmm(ad, bd)
    assert out.dtype == dtype
    ga, gb = torch.autograd.grad(out, (ad, bd), g.to(gpu))
    af, bf = a.float().to(gpu).requires_grad_(True), b.float().to(gpu).requires_grad_(True)
    ref = genbmm.logbmm(af, bf)
    ra, rb = torch.autograd.grad(ref, (af, bf), g.float().to(gpu))
    assert torch.equal(out, ref.to(dtype))
    assert torch.equal(ga, ra.to(dtype)) and torch.equal(gb, rb.to(dtype))
    close(out.float(), oracle.logbmm_grads64(a.float(), b.float(), g.float())[0], rtol=2.0 ** -8, atol=1e-3)


def test_half_inputs_are_twice_differentiable(gpu):
    """float16 / bfloat16 operands stay in their type through forward and backward; the
    double backward widens what the first backward saved, so second-order terms reach the
    half tensors as well."""
    torch.manual_seed(12)
    for dt in (torch.float16, torch.bfloat16):
        a = torch.randn(2, 6, 7).to(dt)
        b = torch.randn(2, 7, 5).to(dt)
        g, u = torch.randn(2, 6, 5).to(dt).float(), torch.randn(2, 6, 7)
        want = oracle.logbmm_second_order64(a.float(), b.float(), g, u, None)
        ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
        out = genbmm.logbmm(ad, bd)
        assert out.dtype == dt
        (ga,) = torch.autograd.grad(out, ad, g.to(gpu).to(dt), create_graph=True)
        assert ga.dtype == dt and ga.requires_grad
        da, db = torch.autograd.grad((ga.float() * u.to(gpu)).sum(), (ad, bd))
        assert da.dtype == dt and float(da.float().abs().max()) > 0 and float(db.float().abs().max()) > 0
        # half rounding of g, of grad_a and of the results: 3 roundings of 2^-8 (bf16) / 2^-11
        tol = 4e-2 if dt == torch.bfloat16 else 6e-3
        close(da.float(), want[0], rtol=tol, atol=tol)
        close(db.float(), want[1], rtol=tol, atol=tol)


# ------------------------------------------------------- streams and HIP graphs
@pytest.mark.parametrize("B,M,K,N", [(5, 33, 70, 129), (32, 256, 128, 256)])
def test_logbmm_on_a_side_stream_and_in_a_graph(gpu, B, M, K, N):
    """The library only enqueues kernels on the stream it is handed (no allocation, no
    synchronisation, no memset): the same calls must give the same bits on a side stream
    and when captured into a HIP graph and replayed, with eager work between replays."""
    lib = _lib.load()
    torch.manual_seed(B + N)
    a, b, g = (torch.randn(s, device=gpu) for s in ((B, M, K), (B, K, N), (B, M, N)))
    p = _lib.ptr

    def buffers():
        return (torch.empty(B, M, N, device=gpu), torch.empty_like(a), torch.empty_like(b),
                torch.empty(lib.genbmm_logbmm_stats_size(B, M, K, N), device=gpu))

    def enqueue(out, ga, gb, stats, stream):
        s = ctypes.c_void_p(stream.cuda_stream)
        assert lib.genbmm_logbmm_fwd(p(a), p(b), p(out), p(stats), B, M, K, N, s) == 0
        assert lib.genbmm_logbmm_bwd(p(a), p(b), p(out), p(g), p(stats), p(ga), p(gb), B, M, K, N, s) == 0

    out0, ga0, gb0, st0 = buffers()
    enqueue(out0, ga0, gb0, st0, torch.cuda.current_stream())
    torch.cuda.synchronize()
    want, wa, wb = oracle.logbmm_grads64(a[:2].cpu(), b[:2].cpu(), g[:2].cpu())
    close(out0[:2], want)
    close(ga0[:2], wa)
    close(gb0[:2], wb)

    side = torch.cuda.Stream()               # default priority
    out1, ga1, gb1, st1 = buffers()
    side.wait_stream(torch.cuda.current_stream())
    enqueue(out1, ga1, gb1, st1, side)
    side.synchronize()
    assert torch.equal(out1, out0) and torch.equal(ga1, ga0) and torch.equal(gb1, gb0)

    out2, ga2, gb2, st2 = buffers()
    graph = torch.cuda.CUDAGraph()
    cap = torch.cuda.Stream()
    cap.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=cap):
        enqueue(out2, ga2, gb2, st2, torch.cuda.current_stream())
    for rep in range(3):
        out2.fill_(float("nan")); ga2.fill_(float("nan")); gb2.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out2, out0) and torch.equal(ga2, ga0) and torch.equal(gb2, gb0), rep
        (a * 2).sum().item()                 # eager work and a sync between replays


def test_maxbmm_and_banded_in_a_graph(gpu):
    lib = _lib.load()
    torch.manual_seed(5)
    B, M, K, N = 4, 40, 50, 36
    a, b = torch.randn(B, M, K, device=gpu), torch.randn(B, K, N, device=gpu)
    out, idx = torch.empty(B, M, N, device=gpu), torch.empty(B, M, N, dtype=torch.int32, device=gpu)
    n, lu, ld = 70, 3, 2
    W = lu + ld + 1
    xa, xb = torch.randn(B, n, W, device=gpu), torch.randn(B, n, W, device=gpu)
    bo = torch.empty(B, n, 2 * W - 1, device=gpu)
    bws = torch.empty(lib.genbmm_banded_workspace_size(lu, ld, lu, ld, B, n), device=gpu)
    p = _lib.ptr

    def enqueue(stream):
        s = ctypes.c_void_p(stream.cuda_stream)
        assert lib.genbmm_maxbmm_fwd(p(a), p(b), p(out), p(idx), B, M, K, N, s) == 0
        assert lib.genbmm_banded_fwd(p(xa), lu, ld, p(xb), lu, ld, p(bo), p(None), p(bws), B, n, 0, s) == 0

    enqueue(torch.cuda.current_stream())
    torch.cuda.synchronize()
    ref = (out.clone(), idx.clone(), bo.clone())
    graph = torch.cuda.CUDAGraph()
    cap = torch.cuda.Stream()
    cap.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=cap):
        enqueue(torch.cuda.current_stream())
    for rep in range(3):
        out.zero_(); idx.zero_(); bo.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref[0]) and torch.equal(idx, ref[1]) and torch.equal(bo, ref[2]), rep
        (a + 1).sum().item()
