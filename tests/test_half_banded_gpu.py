"""float16 / bfloat16 band tensors through the banded entry points (`genbmm_banded_*_f16`,
`_bf16`): the banded kernels compiled for that element type - loads widen, arithmetic and every
workspace are fp32, stores round to nearest.  The contract tested is exact, as for the dense
functions: every result equals what the float entry point returns on the widened tensors,
rounded once (indices identical), for every kernel family a band shape can take; on top of that
the results are compared with the float64 sequential oracle at the tolerance of one rounding of
the output type.  (The reference instantiates its band kernels for Half as well,
banded_cuda_kernel.cu:389, :435, :484, :508, :530, and has no test for it.)"""
import numpy as np
import pytest
import torch

import oracle
from genbmm_amd import _lib
from genbmm_amd.sparse import BandedMatrix, banddiag

pytestmark = pytest.mark.gpu

TYPES = [(torch.float16, "_f16", 2.0 ** -11), (torch.bfloat16, "_bf16", 2.0 ** -8)]
# (n, a_lu, a_ld, b_lu, b_ld): one lane per cell, the memory-fed matrix-core kernels (interior
# and edge tile rows, odd row lengths: rows start at any 2-byte address), whole-strip max,
# strip kernels, bands wider than the matrix, beyond the matrix-core plans
BANDS = [(5, 1, 1, 2, 0), (40, 3, 5, 4, 2), (64, 8, 8, 8, 8), (130, 17, 2, 5, 20), (257, 32, 32, 32, 32),
         (300, 7, 8, 9, 6), (100, 60, 50, 40, 70), (260, 52, 49, 50, 50), (330, 120, 120, 120, 120)]
P = _lib.ptr
LOG, MAX, MUL = 0, 1, 3


def _bands(gpu, dt, n, a_lu, a_ld, b_lu, b_ld, B=3, grid=False):
    def mk(lu, ld):
        x = torch.randn(B, n, n)
        if grid:
            x = torch.round(x * 8) / 8
        return banddiag(x, lu, ld)[0].contiguous().to(gpu).to(dt)
    a, b = mk(a_lu, a_ld), mk(b_lu, b_ld)
    Wo = a.shape[2] + b.shape[2] - 1
    g = torch.randn(B, n, Wo, device=gpu)
    if grid:
        g = (torch.round(g * 8) / 8).clamp(-4, 4)
    return a, b, g.to(dt)


@pytest.mark.parametrize("dt,suffix,eps", TYPES)
@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", BANDS)
@pytest.mark.parametrize("mode,use_ws", [(LOG, True), (LOG, False), (MAX, False), (MUL, False)])
def test_banded_half_equals_float_kernels_rounded(gpu, dt, suffix, eps, n, a_lu, a_ld, b_lu, b_ld, mode, use_ws):
    """use_ws: the log product on its workspace (the others have none)."""
    lib = _lib.load()
    torch.manual_seed(n + mode)
    a, b, g = _bands(gpu, dt, n, a_lu, a_ld, b_lu, b_ld, grid=(mode == MAX))
    B, _, Wa = a.shape
    Wo = g.shape[2]
    a32, b32, g32 = a.float(), b.float(), g.float()
    s = _lib.stream_of(a)
    nws = lib.genbmm_banded_workspace_size(a_lu, a_ld, b_lu, b_ld, B, n) if use_ws else 0
    ws, ws32 = (torch.empty(nws, device=gpu), torch.empty(nws, device=gpu)) if nws else (None, None)
    out, out32 = torch.empty(B, n, Wo, device=gpu, dtype=dt), torch.empty(B, n, Wo, device=gpu)
    idx, idx32 = (torch.empty(B, n, Wo, device=gpu, dtype=torch.int32) for _ in range(2))
    band = (a_lu, a_ld)
    assert getattr(lib, "genbmm_banded_fwd" + suffix)(P(a), *band, P(b), b_lu, b_ld, P(out), P(idx), P(ws), B, n, mode, s) == 0
    assert lib.genbmm_banded_fwd(P(a32), *band, P(b32), b_lu, b_ld, P(out32), P(idx32), P(ws32), B, n, mode, s) == 0
    assert torch.equal(out, out32.to(dt))
    if mode == MAX:
        assert torch.equal(idx, idx32)
    # against the float64 sequential restatement: one rounding of the result on top of the float kernel's error
    want, widx, _ = oracle.seq_band_fwd(a32.cpu().double(), a_lu, a_ld, b32.cpu().double(), b_lu, b_ld, mode, dtype=np.float64)
    err = (out.double().cpu() - want).abs()
    scale = want.abs() if mode != MUL else want.abs() + 4.0 * (Wa ** 0.5)
    assert bool((err <= eps * scale + 1e-4).all()), float(err.max())
    if mode == MAX:
        assert torch.equal(idx.cpu(), widx)
    # backward: the kernels that read `out` read it as stored (rounded); the float kernels get those values
    ga, gb = torch.empty_like(a), torch.empty_like(b)
    ga32, gb32 = torch.empty_like(a32), torch.empty_like(b32)
    oh = out.float()
    nsc = lib.genbmm_banded_scratch_size(a_lu, a_ld, b_lu, b_ld, B, n) if nws else 0
    sc, sc32 = (torch.empty(nsc, device=gpu), torch.empty(nsc, device=gpu)) if nsc else (None, None)
    assert getattr(lib, "genbmm_banded_bwd_scratch" + suffix)(P(a), *band, P(b), b_lu, b_ld, P(out), P(idx), P(ws), P(sc),
                                                             P(g), P(ga), P(gb), B, n, mode, s) == 0
    assert lib.genbmm_banded_bwd_scratch(P(a32), *band, P(b32), b_lu, b_ld, P(oh), P(idx32), P(ws32), P(sc32), P(g32),
                                         P(ga32), P(gb32), B, n, mode, s) == 0
    assert torch.equal(ga, ga32.to(dt)) and torch.equal(gb, gb32.to(dt))
    # the in-place form of the backward gives the same
    ga2, gb2 = torch.empty_like(a), torch.empty_like(b)
    assert getattr(lib, "genbmm_banded_bwd" + suffix)(P(a), *band, P(b), b_lu, b_ld, P(out), P(idx), P(ws), P(g), P(ga2),
                                                     P(gb2), B, n, mode, s) == 0
    assert torch.equal(ga, ga2) and torch.equal(gb, gb2)


@pytest.mark.parametrize("dt,suffix,eps", TYPES)
@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", [(40, 3, 5, 4, 2), (257, 32, 32, 32, 32), (100, 60, 50, 40, 70)])
def test_banded_half_second_order_and_sample(gpu, dt, suffix, eps, n, a_lu, a_ld, b_lu, b_ld):
    lib = _lib.load()
    torch.manual_seed(n)
    a, b, g = _bands(gpu, dt, n, a_lu, a_ld, b_lu, b_ld)
    B, _, Wa = a.shape
    Wo = g.shape[2]
    a32, b32, g32 = a.float(), b.float(), g.float()
    s = _lib.stream_of(a)
    band = (a_lu, a_ld)
    out = torch.empty(B, n, Wo, device=gpu, dtype=dt)
    assert getattr(lib, "genbmm_banded_fwd" + suffix)(P(a), *band, P(b), b_lu, b_ld, P(out), P(None), P(None), B, n, LOG, s) == 0
    oh = out.float()
    ua, ub = torch.randn_like(a32).to(dt), torch.randn_like(b32).to(dt)
    for u_a, u_b in ((ua, ub), (ua, None), (None, ub)):
        da, db, dg = torch.empty_like(a), torch.empty_like(b), torch.empty_like(g)
        t = torch.empty(B, n, Wo, device=gpu)
        assert getattr(lib, "genbmm_banded_bwdbwd" + suffix)(P(a), *band, P(b), b_lu, b_ld, P(out), P(g), P(u_a), P(u_b),
                                                            P(da), P(db), P(dg), P(t), B, n, s) == 0
        da32, db32, dg32 = torch.empty_like(a32), torch.empty_like(b32), torch.empty_like(g32)
        u32 = [None if u is None else u.float() for u in (u_a, u_b)]
        assert lib.genbmm_banded_bwdbwd(P(a32), *band, P(b32), b_lu, b_ld, P(oh), P(g32), P(u32[0]), P(u32[1]),
                                        P(da32), P(db32), P(dg32), B, n, s) == 0
        assert torch.equal(da, da32.to(dt)) and torch.equal(db, db32.to(dt)) and torch.equal(dg, dg32.to(dt))
        assert torch.equal(t, dg32)
    # sample: the same indices as the float function on the widened tensors (with and without workspace)
    for use_ws in (True, False):
        nws = lib.genbmm_banded_workspace_size(a_lu, a_ld, b_lu, b_ld, B, n) if use_ws else 0
        ws, ws32 = (torch.empty(nws, device=gpu), torch.empty(nws, device=gpu)) if nws else (None, None)
        so, so32 = torch.empty(B, n, Wo, device=gpu, dtype=dt), torch.empty(B, n, Wo, device=gpu)
        idx, idx32 = (torch.empty(B, n, Wo, device=gpu, dtype=torch.int32) for _ in range(2))
        assert getattr(lib, "genbmm_banded_sample_fwd" + suffix)(P(a), *band, P(b), b_lu, b_ld, P(so), P(idx), P(ws), 11, 4,
                                                                B, n, s) == 0
        assert lib.genbmm_banded_sample_fwd(P(a32), *band, P(b32), b_lu, b_ld, P(so32), P(idx32), P(ws32), 11, 4, B, n, s) == 0
        assert torch.equal(so, so32.to(dt)) and torch.equal(idx, idx32)


@pytest.mark.parametrize("dt,suffix,eps", TYPES)
def test_banded_half_through_the_public_api(gpu, dt, suffix, eps):
    """BandedMatrix products on half bands return half bands, are differentiable (the log product
    twice) and agree with the float products at the output type's rounding."""
    torch.manual_seed(5)
    n, lu, ld = 96, 9, 7
    a, b, g = _bands(gpu, dt, n, lu, ld, ld, lu)
    X, Y = BandedMatrix(a.clone().requires_grad_(True), lu, ld), BandedMatrix(b.clone().requires_grad_(True), ld, lu)
    Xf = BandedMatrix(a.float().requires_grad_(True), lu, ld)
    Yf = BandedMatrix(b.float().requires_grad_(True), ld, lu)
    for name in ("multiply", "multiply_log", "multiply_max"):
        res, ref = getattr(X, name)(Y), getattr(Xf, name)(Yf)
        assert res.data.dtype == dt and torch.equal(res.data, ref.data.to(dt)), name
        ga, gb = torch.autograd.grad(res.data, (X.data, Y.data), g, create_graph=(name == "multiply_log"))
        ra, rb = torch.autograd.grad(ref.data, (Xf.data, Yf.data), g.float())
        tol = 4 * eps * float(ra.abs().max()) + 1e-3
        assert ga.dtype == dt and float((ga.detach().float() - ra).abs().max()) <= tol, name
        assert float((gb.detach().float() - rb).abs().max()) <= 4 * eps * float(rb.abs().max()) + 1e-3, name
        if name == "multiply_log":
            (da,) = torch.autograd.grad((ga.float() ** 2).sum(), X.data)
            assert da.dtype == dt and bool(torch.isfinite(da.float()).all())
    res = X.multiply_sample(Y, (3, 1))
    assert res.data.dtype == dt
    (gs,) = torch.autograd.grad(res.data.sum(), X.data)
    assert gs.dtype == dt
