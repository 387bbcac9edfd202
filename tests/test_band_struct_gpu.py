"""GPU parity of the band-structure kernels (genbmm_band_shift / _op / _transpose /
_to_dense / _from_dense) against the CPU oracle and the reference's own output vectors.
Data movement: everything is compared bit for bit."""
import operator
import os

import numpy as np
import pytest
import torch

import oracle
from genbmm_amd import _lib
from genbmm_amd.sparse import BandedMatrix, banddiag

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# (batch, n, lu, ld): single column, one-sided bands, bands wider than the matrix, rows
# that are not a multiple of four, and a band too wide for the LDS tile (W > 127)
SHAPES = [(2, 1, 0, 0), (3, 7, 2, 3), (2, 9, 0, 4), (2, 12, 5, 0), (1, 5, 7, 6), (2, 64, 8, 8),
          (3, 130, 17, 2), (2, 257, 32, 32), (1, 300, 70, 90), (2, 96, 100, 101)]


def bits(t):
    return t.detach().cpu().contiguous().view(torch.int32)


def same(got, want):
    assert got.shape == want.shape, (got.shape, want.shape)
    assert torch.equal(bits(got), bits(want))


@pytest.mark.parametrize("case", range(4))
def test_kernels_match_reference_vectors(gpu, case):
    z = np.load(os.path.join(ROOT, "tests", "golden", "band_struct.npz"), allow_pickle=False)
    p = "c%d_" % case
    B, n, lu, ld, olu, old = (int(v) for v in z[p + "meta"])
    fill = float(z[p + "fill"])
    bm = BandedMatrix(torch.from_numpy(z[p + "band"]).to(gpu), lu, ld, fill)
    om = BandedMatrix(torch.from_numpy(z[p + "oband"]).to(gpu), olu, old, fill)

    def check(name, m):
        assert [m.lu, m.ld] == [int(v) for v in z[p + name + "_luld"]], name
        same(m.data, torch.from_numpy(z[p + name]))

    check("band_shift_p1", bm.band_shift(1))
    check("band_shift_m2", bm.band_shift(-2))
    check("band_pad_2", bm.band_pad(2))
    check("band_unshift", bm.band_unshift())
    check("col_shift_p1", bm.col_shift(1))
    check("col_shift_m2", bm.col_shift(-2))
    check("col_unshift", bm.col_unshift())
    check("expand", bm._expand(lu + 2, ld + 1))
    check("op_add", bm.op(om, torch.add, zero=0))              # one pass in the library
    check("op_add", bm.op(om, lambda x, y: x + y, zero=0))     # any callable: torch applies it
    check("op_max", bm.op(om, torch.max, zero=-1e9))
    check("transpose", bm.transpose())
    same(bm.to_dense(), torch.from_numpy(z[p + "to_dense"]))


@pytest.mark.parametrize("batch,n,lu,ld", SHAPES)
def test_kernels_match_oracle(gpu, batch, n, lu, ld):
    torch.manual_seed(n + lu)
    W = lu + ld + 1
    band = torch.randn(batch, n, W)          # every cell distinct, also those outside the matrix
    dev = BandedMatrix(band.to(gpu), lu, ld, fill=-1e9)
    for t in (1, -2, W, -W - 3):
        m = dev.band_shift(t)
        assert (m.lu, m.ld) == (lu + t, ld - t)
        same(m.data, oracle.band_relabel(band, 0, t, W, -1e9))
        m = dev.col_shift(t)
        assert (m.lu, m.ld) == (lu - t, ld + t)
        same(m.data, oracle.band_relabel(band, t, 0, W, -1e9))
    same(dev.band_pad(3).data, oracle.band_relabel(band, 0, -3, W + 6, -1e9))
    same(dev.band_unshift().data, oracle.band_relabel(band, 0, -1, W, -1e9))
    same(dev.col_unshift().data, oracle.band_relabel(band, -1, 0, W, -1e9))
    same(dev._expand(lu + 3, ld + 1).data, oracle.band_relabel(band, 0, -3, W + 4, -1e9))
    same(dev.transpose().data, oracle.band_transpose_indexed(band, lu, ld))
    if n <= 130:
        same(dev.to_dense(), oracle.band_to_dense(band, lu, ld, -1e9))
        dense = torch.randn(batch, n, n)
        got, again = banddiag(dense.to(gpu), lu, ld)
        same(got, oracle.band_from_dense(dense, lu, ld))
        assert again.data_ptr() != 0 and torch.equal(again.cpu(), dense)
        same(dev.transpose().data, oracle.band_transpose(band, lu, ld))
    else:
        # dense forms by index arithmetic in numpy (the loops above are quadratic in n)
        d = band.numpy()
        r = np.arange(n)[:, None]
        c = np.arange(n)[None, :]
        k = r - c + lu
        ok = (k >= 0) & (k < W)
        want = np.where(ok[None], d[:, np.broadcast_to(c, k.shape), np.clip(k, 0, W - 1)], np.float32(-1e9))
        same(dev.to_dense(), torch.from_numpy(want.astype(np.float32)))


@pytest.mark.parametrize("batch,n,lu,ld,olu,old", [(2, 9, 2, 3, 4, 1), (3, 40, 0, 5, 3, 0), (2, 70, 6, 6, 6, 6),
                                                  (1, 33, 1, 9, 8, 2)])
def test_op_kernel_matches_oracle(gpu, batch, n, lu, ld, olu, old):
    torch.manual_seed(n)
    a, b = torch.randn(batch, n, lu + ld + 1), torch.randn(batch, n, olu + old + 1)
    a[0, 0, 0] = float("nan")
    b[-1, -1, -1] = float("nan")
    A, Bm = BandedMatrix(a.to(gpu), lu, ld), BandedMatrix(b.to(gpu), olu, old)
    for fn, ref, zero in ((torch.add, np.add, 0.0), (operator.mul, np.multiply, 1.0),
                          (torch.max, np.maximum, -1e9), (torch.minimum, np.minimum, 1e9)):
        want, wlu, wld = oracle.band_op(a, lu, ld, b, olu, old, ref, zero)
        got = A.op(Bm, fn, zero=zero)
        assert (got.lu, got.ld) == (wlu, wld)
        g, w = got.data.cpu(), want
        assert torch.equal(torch.isnan(g), torch.isnan(w))
        assert torch.equal(bits(torch.nan_to_num(g)), bits(torch.nan_to_num(w)))
        # the same through torch (callable the library does not know)
        other = A.op(Bm, lambda x, y: fn(x, y), zero=zero)
        assert torch.equal(torch.nan_to_num(other.data.cpu()), torch.nan_to_num(w))


def test_structure_kernels_are_differentiable(gpu):
    """The backward of each kernel is its adjoint kernel: gradients equal those of the
    index-arithmetic formulation on the CPU."""
    torch.manual_seed(5)
    n, lu, ld = 37, 4, 2
    band = torch.randn(2, n, lu + ld + 1)

    def run(x, dev):
        m = BandedMatrix(x, lu, ld, fill=-3.0)
        outs = [m.transpose().data, m.band_shift(2).data, m.col_shift(-3).data, m.band_pad(2).data,
                m.to_dense(), m._expand(lu + 1, ld + 2).data, m.band_unshift().data, m.col_unshift().data]
        total = 0
        for i, t in enumerate(outs):
            w = torch.randn(*t.shape, generator=torch.Generator().manual_seed(i)).to(dev)
            total = total + (t * w).sum()
        return torch.autograd.grad(total, x)[0]

    g_cpu = run(band.clone().requires_grad_(True), "cpu")
    g_dev = run(band.to(gpu).requires_grad_(True), gpu)
    assert torch.allclose(g_dev.cpu(), g_cpu, rtol=1e-6, atol=1e-6)
    # banddiag: the gradient is the weight put back on the band's cells of the matrix
    w = torch.randn(2, n, lu + ld + 1)
    xd = torch.randn(2, n, n).to(gpu).requires_grad_(True)
    (gd,) = torch.autograd.grad((banddiag(xd, lu, ld)[0] * w.to(gpu)).sum(), xd)
    same(gd, oracle.band_to_dense(w * oracle.band_from_dense(torch.ones(2, n, n), lu, ld), lu, ld, 0.0))


def test_structure_at_full_size_round_trips(gpu):
    """B=64, n=4096, lu=ld=32: properties that do not need the oracle at this size."""
    torch.manual_seed(7)
    B, n, lu, ld = 64, 4096, 32, 32
    W = lu + ld + 1
    data = torch.rand(B, n, W, device=gpu) * 2 - 1
    m = BandedMatrix(data, lu, ld)
    inside = banddiag(torch.ones(1, n, n, device=gpu), lu, ld)[0] > 0   # cells inside the matrix
    t = m.transpose()
    tt = t.transpose()
    assert torch.equal(tt.data, torch.where(inside, data, torch.zeros((), device=gpu)))
    # transpose against the dense definition on a batch subset
    sub = BandedMatrix(data[:2].contiguous(), lu, ld)
    dense = sub.to_dense()
    assert torch.equal(banddiag(dense.transpose(-2, -1).contiguous(), ld, lu)[0], t.data[:2])
    assert torch.equal(banddiag(dense, lu, ld)[0], torch.where(inside, data[:2], torch.zeros((), device=gpu)))
    # shifts undo each other away from the cells they push out
    s = m.band_shift(3).band_shift(-3)
    assert torch.equal(s.data[:, :, 3:], data[:, :, 3:]) and bool((s.data[:, :, :3] == 0).all())
    c = m.col_shift(5).col_shift(-5)
    assert torch.equal(c.data[:, 5:], data[:, 5:]) and bool((c.data[:, :5] == 0).all())
    # through the C ABI directly, on the side of the Python layer
    out = torch.empty_like(data)
    rc = _lib.load().genbmm_band_transpose(_lib.ptr(data), _lib.ptr(out), B, n, lu, ld, _lib.stream_of(data))
    assert rc == 0 and torch.equal(out, t.data)


def test_structure_argument_errors(gpu):
    lib = _lib.load()
    x = torch.zeros(2, 4, 3, device=gpu)
    s = _lib.stream_of(x)
    assert lib.genbmm_band_transpose(_lib.ptr(x), _lib.ptr(x), 2, 4, -1, 3, s) < 0
    assert lib.genbmm_band_transpose(_lib.ptr(None), _lib.ptr(x), 2, 4, 1, 1, s) < 0
    assert lib.genbmm_band_shift(_lib.ptr(x), _lib.ptr(x), 2, 4, 3, 0, 0, 0, 0.0, s) < 0
    assert lib.genbmm_band_op(_lib.ptr(x), 1, 1, _lib.ptr(x), 1, 1, _lib.ptr(x), 2, 4, 9, 0.0, s) < 0
    assert lib.genbmm_band_to_dense(_lib.ptr(x), _lib.ptr(None), 2, 4, 1, 1, 0.0, s) < 0
    assert lib.genbmm_band_from_dense(_lib.ptr(x), _lib.ptr(x), 0, 4, 4, 1, 1, s) == 0   # empty batch
