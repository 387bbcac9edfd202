"""GPU parity of the banded (+,x) and log products on the bands that the matrix-core
kernels take (from 3 diagonals on, up to about 160 in the result): edges of the matrix
inside a tile row, tile rows cut by n, one-sided bands, the widest first operands,
operands that do not start on 16 bytes, values that are not finite.  All against the float64 sequential restatement of the reference
kernel (oracle.seq_band_fwd / seq_band_bwd)."""
import numpy as np
import pytest
import torch

import oracle
from genbmm_amd.sparse import BandedMatrix, banddiag

pytestmark = pytest.mark.gpu

# (n, a_lu, a_ld, b_lu, b_ld)
WIDE = [(300, 12, 12, 12, 12), (95, 20, 9, 14, 16), (513, 32, 32, 32, 32), (64, 30, 0, 0, 30),
        (33, 16, 16, 16, 16), (1000, 3, 30, 28, 2), (129, 4, 4, 20, 20), (40, 28, 28, 30, 30),
        (257, 0, 31, 31, 0), (70, 10, 5, 3, 8), (400, 40, 40, 40, 40), (210, 0, 60, 60, 0),
        (150, 70, 0, 2, 1), (47, 1, 1, 1, 1)]


def close(x, ref, rtol=1e-5, atol=1e-5):
    x, ref = x.detach().cpu().double(), ref.detach().cpu().double()
    assert torch.allclose(x, ref, rtol=rtol, atol=atol, equal_nan=True), float((x - ref).abs().nan_to_num().max())


def pair(n, a_lu, a_ld, b_lu, b_ld, batch=2):
    a = banddiag(torch.randn(batch, n, n), a_lu, a_ld)[0].contiguous()
    b = banddiag(torch.randn(batch, n, n), b_lu, b_ld)[0].contiguous()
    return a, b


def offset_copy(t, gpu, shift):
    """The same values in device memory that starts `shift` floats past a 16-byte boundary."""
    flat = torch.empty(t.numel() + 8, device=gpu)
    view = flat[shift:shift + t.numel()].view(t.shape)
    view.copy_(t)
    assert view.data_ptr() % 16 == 4 * (shift % 4) and view.is_contiguous()
    return view


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", WIDE)
@pytest.mark.parametrize("mode", [0, 3])
def test_wide_bands_forward_backward(gpu, n, a_lu, a_ld, b_lu, b_ld, mode):
    torch.manual_seed(n + 31 * mode)
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld)
    W = a.shape[2] + b.shape[2] - 1
    g = torch.randn(2, n, W)
    X = BandedMatrix(a.to(gpu).requires_grad_(True), a_lu, a_ld)
    Y = BandedMatrix(b.to(gpu).requires_grad_(True), b_lu, b_ld)
    res = (X.multiply_log if mode == 0 else X.multiply)(Y)
    want, _, _ = oracle.seq_band_fwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, mode, dtype=np.float64)
    close(res.data, want)
    ga, gb = torch.autograd.grad(res.data, (X.data, Y.data), g.to(gpu))
    wa, wb = oracle.seq_band_bwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, g.double(), mode, dtype=np.float64)
    close(ga, wa)
    close(gb, wb)


@pytest.mark.parametrize("shift", [1, 2, 3])
@pytest.mark.parametrize("mode", [0, 3])
def test_operands_off_the_16_byte_grid(gpu, shift, mode):
    n, a_lu, a_ld, b_lu, b_ld = 150, 13, 14, 15, 12
    torch.manual_seed(shift)
    a, b = pair(n, a_lu, a_ld, b_lu, b_ld)
    g = torch.randn(2, n, a.shape[2] + b.shape[2] - 1)
    ad = offset_copy(a, gpu, shift).requires_grad_(True)
    bd = offset_copy(b, gpu, shift + 1).requires_grad_(True)
    X, Y = BandedMatrix(ad, a_lu, a_ld), BandedMatrix(bd, b_lu, b_ld)
    res = (X.multiply_log if mode == 0 else X.multiply)(Y)
    want, _, _ = oracle.seq_band_fwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, mode, dtype=np.float64)
    close(res.data, want)
    ga, gb = torch.autograd.grad(res.data, (ad, bd), offset_copy(g, gpu, shift + 2))
    wa, wb = oracle.seq_band_bwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, g.double(), mode, dtype=np.float64)
    close(ga, wa)
    close(gb, wb)


def test_values_that_are_not_finite(gpu):
    """inf and NaN in an operand reach exactly the cells the reference lets them reach: a
    strip that holds one is computed cell by cell."""
    n, lu, ld = 200, 14, 15
    torch.manual_seed(5)
    a, b = pair(n, lu, ld, ld, lu)
    a[0, 40, 3] = float("inf")
    a[1, 101, 7] = float("nan")
    b[0, 77, 20] = -float("inf")
    b[1, 150, 0] = float("inf")
    ad, bd = a.to(gpu), b.to(gpu)
    res = BandedMatrix(ad, lu, ld).multiply(BandedMatrix(bd, ld, lu))
    want, _, _ = oracle.seq_band_fwd(a.double(), lu, ld, b.double(), ld, lu, 3, dtype=np.float64)
    got = res.data.cpu().double()
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    assert torch.equal(torch.isinf(got), torch.isinf(want))
    close(got.nan_to_num(posinf=0.0, neginf=0.0), want.nan_to_num(posinf=0.0, neginf=0.0))
    # gradients with a finite g: rows away from the special values are untouched by them
    g = torch.randn(2, n, res.data.shape[2])
    ar, br = ad.clone().requires_grad_(True), bd.clone().requires_grad_(True)
    out = BandedMatrix(ar, lu, ld).multiply(BandedMatrix(br, ld, lu))
    ga, gb = torch.autograd.grad(out.data, (ar, br), g.to(gpu))
    wa, wb = oracle.seq_band_bwd(a.double(), lu, ld, b.double(), ld, lu, g.double(), 3, dtype=np.float64)
    for got_g, want_g in ((ga, wa), (gb, wb)):
        got_g = got_g.cpu().double()
        fin = torch.isfinite(want_g)
        assert torch.equal(torch.isfinite(got_g), fin)
        close(got_g[fin], want_g[fin])


def test_log_product_with_masked_and_infinite_cells(gpu):
    n, lu, ld = 160, 16, 16
    torch.manual_seed(9)
    a, b = pair(n, lu, ld, ld, lu)
    a[0, 10:60, 5:9] = -float("inf")
    b[1, 90, :] = -float("inf")       # a fully masked row
    a[1, 120, 2] = float("inf")
    ad, bd = a.to(gpu).requires_grad_(True), b.to(gpu).requires_grad_(True)
    res = BandedMatrix(ad, lu, ld).multiply_log(BandedMatrix(bd, ld, lu))
    want, _, _ = oracle.seq_band_fwd(a.double(), lu, ld, b.double(), ld, lu, 0, dtype=np.float64)
    got = res.data.detach().cpu().double()
    assert torch.equal(torch.isfinite(got), torch.isfinite(want))
    fin = torch.isfinite(want)
    close(got[fin], want[fin])
    assert torch.equal(got[~fin].nan_to_num(nan=7.0), want[~fin].nan_to_num(nan=7.0))


def test_random_bands_against_the_oracle(gpu):
    """Seeded sweep over band shapes around the kernels' switching points (4, 8, 25
    diagonals; strips of 32 and 64 rows; tiles of 16): forward and both gradients of the
    (+,x) and the log product."""
    rng = np.random.default_rng(20240607)
    for case in range(36):
        a_lu, a_ld, b_lu, b_ld = (int(v) for v in rng.integers(0, 19, size=4))
        if case % 3 == 0:  # keep some operands on the narrow side
            a_lu, a_ld = a_lu % 4, a_ld % 3
        n = int(rng.choice([1, 2, 7, 15, 16, 17, 31, 32, 33, 63, 64, 65, 97, 128, 131, 200]))
        mode = 0 if case % 2 else 3
        torch.manual_seed(case)
        a, b = pair(n, a_lu, a_ld, b_lu, b_ld)
        W = a.shape[2] + b.shape[2] - 1
        g = torch.randn(2, n, W)
        X = BandedMatrix(a.to(gpu).requires_grad_(True), a_lu, a_ld)
        Y = BandedMatrix(b.to(gpu).requires_grad_(True), b_lu, b_ld)
        res = (X.multiply_log if mode == 0 else X.multiply)(Y)
        want, _, _ = oracle.seq_band_fwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, mode, dtype=np.float64)
        tag = (case, n, a_lu, a_ld, b_lu, b_ld, mode)
        assert torch.allclose(res.data.detach().cpu().double(), want, rtol=1e-5, atol=1e-5), tag
        ga, gb = torch.autograd.grad(res.data, (X.data, Y.data), g.to(gpu))
        wa, wb = oracle.seq_band_bwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, g.double(), mode,
                                     dtype=np.float64)
        assert torch.allclose(ga.cpu().double(), wa, rtol=1e-5, atol=1e-5), tag
        assert torch.allclose(gb.cpu().double(), wb, rtol=1e-5, atol=1e-5), tag


def test_random_bands_max_product_bit_exact(gpu):
    """The whole-strip max-plus forward against the oracle, values on a grid of 1/8 so that
    ties occur: values, arg-max indices (through the C ABI) and gradients must be equal."""
    from genbmm_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(77)
    for case in range(24):
        a_lu, a_ld, b_lu, b_ld = (int(v) for v in rng.integers(0, 21, size=4))
        if case % 4 == 0:
            b_lu, b_ld = b_lu % 5, b_ld % 4
        n = int(rng.choice([3, 16, 33, 63, 64, 65, 100, 128, 150, 257]))
        torch.manual_seed(100 + case)
        grid = lambda *s: torch.round(torch.randn(*s) * 8) / 8
        a = banddiag(grid(2, n, n), a_lu, a_ld)[0].contiguous()
        b = banddiag(grid(2, n, n), b_lu, b_ld)[0].contiguous()
        W = a.shape[2] + b.shape[2] - 1
        ad, bd = a.to(gpu), b.to(gpu)
        out = torch.empty(2, n, W, device=gpu)
        idx = torch.empty(2, n, W, dtype=torch.int32, device=gpu)
        rc = lib.genbmm_banded_fwd(_lib.ptr(ad), a_lu, a_ld, _lib.ptr(bd), b_lu, b_ld, _lib.ptr(out), _lib.ptr(idx),
                                   _lib.ptr(None), 2, n, 1, _lib.stream_of(ad))
        assert rc == 0
        want, widx, _ = oracle.seq_band_fwd(a, a_lu, a_ld, b, b_lu, b_ld, 1)
        tag = (case, n, a_lu, a_ld, b_lu, b_ld)
        assert torch.equal(out.cpu(), want), tag
        assert torch.equal(idx.cpu(), widx), tag
        g = grid(2, n, W).clamp(-4, 4)
        X = BandedMatrix(ad.clone().requires_grad_(True), a_lu, a_ld)
        Y = BandedMatrix(bd.clone().requires_grad_(True), b_lu, b_ld)
        res = X.multiply_max(Y)
        ga, gb = torch.autograd.grad(res.data, (X.data, Y.data), g.to(gpu))
        wa, wb = oracle.seq_band_bwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, g.double(), 1, dtype=np.float64)
        assert torch.equal(ga.cpu().double(), wa) and torch.equal(gb.cpu().double(), wb), tag


def _max_through_abi(gpu, ad, bd, a_lu, a_ld, b_lu, b_ld):
    from genbmm_amd import _lib
    lib = _lib.load()
    B, n = ad.shape[0], ad.shape[1]
    W = ad.shape[2] + bd.shape[2] - 1
    out = torch.empty(B, n, W, device=gpu)
    idx = torch.empty(B, n, W, dtype=torch.int32, device=gpu)
    rc = lib.genbmm_banded_fwd(_lib.ptr(ad), a_lu, a_ld, _lib.ptr(bd), b_lu, b_ld, _lib.ptr(out), _lib.ptr(idx),
                               _lib.ptr(None), B, n, 1, _lib.stream_of(ad))
    assert rc == 0
    return out, idx


@pytest.mark.parametrize("shift", [1, 2, 3])
def test_max_product_operands_off_the_16_byte_grid(gpu, shift):
    """The whole-strip max-plus forward on operands that start 4, 8, 12 bytes past a 16-byte
    boundary (its flat copy into LDS then has a lead), values and indices bit-exact."""
    n, a_lu, a_ld, b_lu, b_ld = 150, 13, 14, 15, 12
    torch.manual_seed(40 + shift)
    grid = lambda *s: torch.round(torch.randn(*s) * 8) / 8
    a = banddiag(grid(2, n, n), a_lu, a_ld)[0].contiguous()
    b = banddiag(grid(2, n, n), b_lu, b_ld)[0].contiguous()
    out, idx = _max_through_abi(gpu, offset_copy(a, gpu, shift), offset_copy(b, gpu, shift + 1), a_lu, a_ld, b_lu, b_ld)
    want, widx, _ = oracle.seq_band_fwd(a, a_lu, a_ld, b, b_lu, b_ld, 1)
    assert torch.equal(out.cpu(), want) and torch.equal(idx.cpu(), widx)


def test_max_product_values_that_are_not_finite(gpu):
    """+-inf and NaN operands next to the -inf padding between the staged rows of b: the same
    cells become non-finite as in the oracle's walk, the same k wins everywhere (NaN never
    wins a strict '>'; -inf + inf is NaN)."""
    n, lu, ld = 200, 14, 15
    torch.manual_seed(6)
    a, b = pair(n, lu, ld, ld, lu)
    a[0, 40, 3] = float("inf")
    a[1, 101, 7] = float("nan")
    b[0, 77, 20] = -float("inf")
    b[1, 150, 0] = float("inf")
    a[1, 30, :] = -float("inf")
    for shift in (0, 1):
        ad = offset_copy(a, gpu, shift) if shift else a.to(gpu)
        out, idx = _max_through_abi(gpu, ad, b.to(gpu), lu, ld, ld, lu)
        want, widx, _ = oracle.seq_band_fwd(a, lu, ld, b, ld, lu, 1)
        assert torch.equal(out.cpu().view(torch.int32), want.view(torch.int32))
        assert torch.equal(idx.cpu(), widx)


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", [(700, 75, 74, 4, 3), (513, 60, 60, 12, 12), (330, 0, 139, 10, 0)])
def test_max_product_on_the_widest_whole_strip_bands(gpu, n, a_lu, a_ld, b_lu, b_ld):
    """Result bands of 145 to 157 diagonals (twenty blocks of eight per row, the fifth block
    of the waves in use; a wide first operand against a narrow second keeps the tiles within
    the kernel's LDS budget) on matrices long enough for interior strips."""
    torch.manual_seed(n)
    grid = lambda *s: torch.round(torch.randn(*s) * 8) / 8
    a = banddiag(grid(2, n, n), a_lu, a_ld)[0].contiguous()
    b = banddiag(grid(2, n, n), b_lu, b_ld)[0].contiguous()
    out, idx = _max_through_abi(gpu, a.to(gpu), b.to(gpu), a_lu, a_ld, b_lu, b_ld)
    want, widx, _ = oracle.seq_band_fwd(a, a_lu, a_ld, b, b_lu, b_ld, 1)
    assert torch.equal(out.cpu(), want) and torch.equal(idx.cpu(), widx)
