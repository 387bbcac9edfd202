"""GPU parity of the forward of the banded (+,x) and log products on the bands that the block
kernel takes (about 53 to 65 diagonals per operand; csrc/banded_block.h): workgroups that walk
several 32-row steps, an odd and an even number of them, rows cut by n inside a step, a single
batch item (loads next to both ends of the tensors), one-sided and unequal bands, the variant
with seven slabs per block, operands too small to come apart into three bfloat16 parts exactly,
values that are not finite, and float16 / bfloat16 bands.  All against the float64 sequential
restatement of the reference kernel (oracle.seq_band_fwd); the gradients of the same shapes go
through the kernels that tests/test_banded_mfma_gpu.py covers and are checked here as well."""
import numpy as np
import pytest
import torch

import oracle
from genbmm_amd import _lib
from genbmm_amd.sparse import BandedMatrix, banddiag

pytestmark = pytest.mark.gpu
P = _lib.ptr

# (batch, n, a_lu, a_ld, b_lu, b_ld)
SHAPES = [
    (2, 257, 32, 32, 32, 32),    # one step per workgroup, the last one cut by n
    (1, 70, 30, 30, 28, 28),     # one item: the first and the last block lie at the tensors' ends
    (1, 33, 32, 32, 32, 32),     # band wider than the matrix
    (40, 640, 32, 32, 32, 32),   # three steps per workgroup (and a last workgroup with two)
    (24, 1000, 26, 26, 30, 30),  # steps cut by n, four steps per workgroup at the end
    (70, 1500, 32, 32, 32, 32),  # twelve steps per workgroup
    (3, 300, 64, 0, 0, 64),      # one-sided bands
    (3, 300, 0, 56, 60, 0),
    (2, 200, 40, 29, 26, 26),    # seven slabs in a block of the first operand
    (2, 260, 20, 33, 40, 14),
    (3, 129, 27, 27, 32, 32),
]


def close(x, ref, rtol=1e-5, atol=1e-5):
    x, ref = x.detach().cpu().double(), ref.detach().cpu().double()
    assert torch.allclose(x, ref, rtol=rtol, atol=atol, equal_nan=True), float((x - ref).abs().nan_to_num().max())


def pair(batch, n, a_lu, a_ld, b_lu, b_ld):
    a = banddiag(torch.randn(batch, n, n), a_lu, a_ld)[0].contiguous()
    b = banddiag(torch.randn(batch, n, n), b_lu, b_ld)[0].contiguous()
    return a, b


@pytest.mark.parametrize("batch,n,a_lu,a_ld,b_lu,b_ld", SHAPES)
@pytest.mark.parametrize("mode", [0, 3])
def test_block_kernel_forward_and_gradients(gpu, batch, n, a_lu, a_ld, b_lu, b_ld, mode):
    torch.manual_seed(n + 7 * mode)
    a, b = pair(batch, n, a_lu, a_ld, b_lu, b_ld)
    # cells of the band outside the matrix hold anything: the product must not read them
    a[:, :3, :] += 100.0 * (a[:, :3, :] == 0)
    b[:, -3:, :] += 100.0 * (b[:, -3:, :] == 0)
    W = a.shape[2] + b.shape[2] - 1
    X = BandedMatrix(a.to(gpu).requires_grad_(True), a_lu, a_ld)
    Y = BandedMatrix(b.to(gpu).requires_grad_(True), b_lu, b_ld)
    res = (X.multiply_log if mode == 0 else X.multiply)(Y)
    want, _, _ = oracle.seq_band_fwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, mode, dtype=np.float64)
    close(res.data, want)
    if batch * n <= 8000:
        g = torch.randn(batch, n, W)
        ga, gb = torch.autograd.grad(res.data, (X.data, Y.data), g.to(gpu))
        wa, wb = oracle.seq_band_bwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, g.double(), mode, dtype=np.float64)
        close(ga, wa)
        close(gb, wb)


def test_block_kernel_operands_below_the_three_part_range(gpu):
    """A float below about 2^-100 does not come apart into three bfloat16 parts exactly; a
    workgroup that meets one computes its rows cell by cell instead."""
    batch, n, lu = 3, 200, 32
    torch.manual_seed(11)
    a, b = pair(batch, n, lu, lu, lu, lu)
    a[1, 50:60, :] *= 1e-33
    b[1, 40:80, :] *= 1e30           # products of about 1e-3: the small operands matter
    b[2, 100, 7] = 3e-39             # a subnormal of the operand type's
    got = BandedMatrix(a.to(gpu), lu, lu).multiply(BandedMatrix(b.to(gpu), lu, lu)).data
    want, _, _ = oracle.seq_band_fwd(a.double(), lu, lu, b.double(), lu, lu, 3, dtype=np.float64)
    got, want = got.cpu().double(), want.double()
    # every cell to 1e-5 of the sum of its terms' magnitudes (its own scale: cells of the small rows of
    # a against the large rows of b are about 1e-3, their neighbours 1e-33 and 1e+30)
    scale, _, _ = oracle.seq_band_fwd(a.double().abs(), lu, lu, b.double().abs(), lu, lu, 3, dtype=np.float64)
    assert bool(((got - want).abs() <= 1e-5 * scale.double()).all())
    assert 1e-4 < float(want[1, 50:60].abs().max()) < 1.0


def test_block_kernel_values_that_are_not_finite(gpu):
    batch, n, lu = 2, 300, 32
    torch.manual_seed(5)
    a, b = pair(batch, n, lu, lu, lu, lu)
    a[0, 40, 3] = float("inf")
    a[1, 101, 7] = float("nan")
    b[0, 77, 20] = -float("inf")
    b[1, 150, 0] = float("inf")
    a[1, 200, 10] = 3.0e38           # rounds to infinity as a bfloat16
    res = BandedMatrix(a.to(gpu), lu, lu).multiply(BandedMatrix(b.to(gpu), lu, lu))
    want, _, _ = oracle.seq_band_fwd(a.double(), lu, lu, b.double(), lu, lu, 3, dtype=np.float32)
    got, want = res.data.cpu().double(), want.double()
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    assert torch.equal(torch.isinf(got), torch.isinf(want))
    close(got.nan_to_num(posinf=0.0, neginf=0.0), want.nan_to_num(posinf=0.0, neginf=0.0))


def test_block_kernel_log_product_with_masked_cells(gpu):
    batch, n, lu = 2, 260, 30
    torch.manual_seed(9)
    a, b = pair(batch, n, lu, lu, lu, lu)
    a[0, 10:60, 5:9] = -float("inf")
    b[1, 90, :] = -float("inf")      # a fully masked row
    a[1, 120, 2] = float("inf")
    a[0, 200:230, :] -= 200.0        # sums far below the guard of the factored form
    ad, bd = a.to(gpu), b.to(gpu)
    res = BandedMatrix(ad, lu, lu).multiply_log(BandedMatrix(bd, lu, lu))
    want, _, _ = oracle.seq_band_fwd(a.double(), lu, lu, b.double(), lu, lu, 0, dtype=np.float64)
    got = res.data.detach().cpu().double()
    assert torch.equal(torch.isfinite(got), torch.isfinite(want))
    fin = torch.isfinite(want)
    close(got[fin], want[fin])
    assert torch.equal(got[~fin].nan_to_num(nan=7.0), want[~fin].nan_to_num(nan=7.0))


@pytest.mark.parametrize("dt,suffix,eps", [(torch.float16, "_f16", 2.0 ** -11), (torch.bfloat16, "_bf16", 2.0 ** -8)])
@pytest.mark.parametrize("mode", [0, 3])
def test_block_kernel_half_bands(gpu, dt, suffix, eps, mode):
    """Several steps per workgroup on float16 / bfloat16 bands: equal to the float entry point on
    the widened bands, rounded once."""
    lib = _lib.load()
    batch, n, lu = 40, 640, 32
    torch.manual_seed(3)
    a, b = (t.to(gpu).to(dt) for t in pair(batch, n, lu, lu, lu, lu))
    Wo = a.shape[2] + b.shape[2] - 1
    s = _lib.stream_of(a)
    nws = lib.genbmm_banded_workspace_size(lu, lu, lu, lu, batch, n)
    ws, ws32 = torch.empty(nws, device=gpu), torch.empty(nws, device=gpu)
    out, out32 = torch.empty(batch, n, Wo, device=gpu, dtype=dt), torch.empty(batch, n, Wo, device=gpu)
    a32, b32 = a.float(), b.float()
    assert getattr(lib, "genbmm_banded_fwd" + suffix)(P(a), lu, lu, P(b), lu, lu, P(out), None, P(ws), batch, n, mode, s) == 0
    assert lib.genbmm_banded_fwd(P(a32), lu, lu, P(b32), lu, lu, P(out32), None, P(ws32), batch, n, mode, s) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, out32.to(dt))
    want, _, _ = oracle.seq_band_fwd(a32.cpu().double(), lu, lu, b32.cpu().double(), lu, lu, mode, dtype=np.float64)
    close(out.float(), want, rtol=2 * eps, atol=2 * eps)
