"""The torch.library operators (genbmm_amd.ops): same results as the autograd Functions,
registrations that pass torch's operator checks, and graphs that trace and differentiate
under torch.compile (backend "aot_eager": capture and functionalisation, no code generation)."""
import pytest
import torch

import genbmm_amd as genbmm
from genbmm_amd import ops

pytestmark = pytest.mark.gpu


def pair(gpu, B=3, M=70, K=45, N=66, grid=False):
    torch.manual_seed(M)
    mk = (lambda *s: torch.round(torch.randn(*s) * 8) / 8) if grid else torch.randn
    return mk(B, M, K).to(gpu).requires_grad_(True), mk(B, K, N).to(gpu).requires_grad_(True)


def test_operators_match_the_functions(gpu):
    a, b = pair(gpu)
    g = torch.randn(3, 70, 66, device=gpu)
    for op, fn in ((ops.logbmm, genbmm.logbmm), (ops.maxbmm, genbmm.maxbmm), (ops.prodmaxbmm, genbmm.prodmaxbmm)):
        y, want = op(a, b), fn(a, b)
        assert torch.equal(y, want)
        ga, gb = torch.autograd.grad(y, (a, b), g)
        wa, wb = torch.autograd.grad(want, (a, b), g)
        assert torch.equal(ga, wa) and torch.equal(gb, wb)
    y = ops.samplebmm(a, b, 1234, 8)
    want = genbmm.samplebmm(a, b, (1234, 8))
    assert torch.equal(y, want)
    assert torch.equal(torch.autograd.grad(y, a, g)[0], torch.autograd.grad(want, a, g)[0])
    # logbmm twice
    u = torch.randn_like(a)
    for op in (ops.logbmm, genbmm.logbmm):
        (ga,) = torch.autograd.grad(op(a, b), a, g, create_graph=True)
        r = torch.autograd.grad((ga * u).sum(), (a, b))
        if op is ops.logbmm:
            first = r
    assert torch.equal(first[0], r[0]) and torch.equal(first[1], r[1])


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_operators_on_half_tensors(gpu, dt):
    """float16 / bfloat16 tensors: the operators and the autograd Functions call the same
    entry points (same bits), the registrations pass torch's checks, a graph compiles."""
    a, b = pair(gpu)
    a, b = a.detach().to(dt).requires_grad_(True), b.detach().to(dt).requires_grad_(True)
    g = torch.randn(3, 70, 66, device=gpu).to(dt)
    for op, fn in ((ops.logbmm, genbmm.logbmm), (ops.maxbmm, genbmm.maxbmm), (ops.prodmaxbmm, genbmm.prodmaxbmm)):
        y, want = op(a, b), fn(a, b)
        assert y.dtype == dt and torch.equal(y, want)
        ga, gb = torch.autograd.grad(y, (a, b), g)
        wa, wb = torch.autograd.grad(want, (a, b), g)
        assert ga.dtype == dt and torch.equal(ga, wa) and torch.equal(gb, wb)
    assert torch.equal(ops.samplebmm(a, b, 99, 4), genbmm.samplebmm(a, b, (99, 4)))
    u = torch.randn_like(a)
    res = []
    for op in (ops.logbmm, genbmm.logbmm):
        (ga,) = torch.autograd.grad(op(a, b), a, g, create_graph=True)
        res.append(torch.autograd.grad((ga * u).sum(), (a, b)))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])
    ad, bd = a.detach()[:, :9, :12].contiguous(), b.detach()[:, :12, :7].contiguous()
    tests = ("test_schema", "test_faketensor", "test_autograd_registration")
    torch.library.opcheck(torch.ops.genbmm_amd.logbmm_fwd.default, (ad, bd), test_utils=tests)
    torch.library.opcheck(torch.ops.genbmm_amd.prodmaxbmm_fwd.default, (ad, bd), test_utils=tests)
    out, stats = torch.ops.genbmm_amd.logbmm_fwd(ad, bd)
    torch.library.opcheck(torch.ops.genbmm_amd.logbmm_bwd.default, (ad, bd, out, torch.randn_like(out), stats),
                          test_utils=tests)
    compiled = torch.compile(lambda x, y: ops.logbmm(x, y).float().sum(), backend="aot_eager", fullgraph=True)
    assert torch.equal(compiled(a, b), genbmm.logbmm(a, b).float().sum())


def test_registrations_pass_opcheck(gpu):
    a, b = pair(gpu, 2, 9, 12, 7)
    ad, bd = a.detach(), b.detach()
    tests = ("test_schema", "test_faketensor", "test_autograd_registration")
    torch.library.opcheck(torch.ops.genbmm_amd.logbmm_fwd.default, (ad, bd), test_utils=tests)
    torch.library.opcheck(torch.ops.genbmm_amd.maxbmm_fwd.default, (ad, bd), test_utils=tests)
    torch.library.opcheck(torch.ops.genbmm_amd.prodmaxbmm_fwd.default, (ad, bd), test_utils=tests)
    torch.library.opcheck(torch.ops.genbmm_amd.samplebmm_fwd.default, (ad, bd, 5, 0), test_utils=tests)
    out, idx = torch.ops.genbmm_amd.maxbmm_fwd(ad, bd)
    g = torch.randn_like(out)
    torch.library.opcheck(torch.ops.genbmm_amd.argmax_bwd.default, (idx, g, 12), test_utils=tests)
    _, idx, factors = torch.ops.genbmm_amd.prodmaxbmm_fwd(ad, bd)
    torch.library.opcheck(torch.ops.genbmm_amd.prodmax_bwd.default, (idx, factors, g, 12), test_utils=tests)
    # the backward operators declare no mutation: the forward's workspace is only read
    # (checked by test_schema), on a small shape and on one that runs on the matrix cores
    for a2, b2 in ((ad, bd), (torch.randn(2, 128, 32, device=gpu), torch.randn(2, 32, 128, device=gpu))):
        out, stats = torch.ops.genbmm_amd.logbmm_fwd(a2, b2)
        g = torch.randn_like(out)
        torch.library.opcheck(torch.ops.genbmm_amd.logbmm_bwd.default, (a2, b2, out, g, stats), test_utils=tests)
        torch.library.opcheck(torch.ops.genbmm_amd.logbmm_bwdbwd.default,
                              (a2, b2, out, g, torch.randn_like(a2), torch.randn_like(b2)), test_utils=tests)


def test_graphs_compile_and_differentiate(gpu):
    a, b = pair(gpu, 2, 40, 33, 48)

    def chain(x, y):
        z = ops.logbmm(x, y)                       # (2, 40, 48)
        w = ops.maxbmm(z, y.transpose(1, 2).contiguous())   # (2, 40, 33)
        return (w * w).sum() + ops.prodmaxbmm(x.abs(), y.abs()).sum()

    want = chain(a, b)
    wa, wb = torch.autograd.grad(want, (a, b))
    compiled = torch.compile(chain, backend="aot_eager", fullgraph=True)
    got = compiled(a, b)
    ga, gb = torch.autograd.grad(got, (a, b))
    assert torch.equal(got, want) and torch.equal(ga, wa) and torch.equal(gb, wb)


def band_pair(gpu, n=90, a_lu=9, a_ld=4, b_lu=6, b_ld=11, grid=False):
    from genbmm_amd.sparse import banddiag
    torch.manual_seed(n)
    mk = (lambda *s: torch.round(torch.randn(*s) * 8) / 8) if grid else torch.randn
    a = banddiag(mk(2, n, n), a_lu, a_ld)[0].contiguous().to(gpu).requires_grad_(True)
    b = banddiag(mk(2, n, n), b_lu, b_ld)[0].contiguous().to(gpu).requires_grad_(True)
    return a, b, (a_lu, a_ld, b_lu, b_ld)


def test_banded_operators_match_the_band_matrix_methods(gpu):
    from genbmm_amd.sparse import BandedMatrix
    for grid, op, name in ((False, ops.banded_multiply, "multiply"), (False, ops.banded_multiply_log, "multiply_log"),
                           (True, ops.banded_multiply_max, "multiply_max")):
        a, b, (a_lu, a_ld, b_lu, b_ld) = band_pair(gpu, grid=grid)
        y = op(a, a_lu, a_ld, b, b_lu, b_ld)
        want = getattr(BandedMatrix(a, a_lu, a_ld), name)(BandedMatrix(b, b_lu, b_ld)).data
        assert torch.equal(y, want)
        g = torch.randn_like(y)
        ga, gb = torch.autograd.grad(y, (a, b), g)
        wa, wb = torch.autograd.grad(want, (a, b), g)
        assert torch.equal(ga, wa) and torch.equal(gb, wb)
    # the log product twice
    a, b, (a_lu, a_ld, b_lu, b_ld) = band_pair(gpu)
    u = torch.randn_like(a)
    res = []
    for f in (lambda: ops.banded_multiply_log(a, a_lu, a_ld, b, b_lu, b_ld),
              lambda: BandedMatrix(a, a_lu, a_ld).multiply_log(BandedMatrix(b, b_lu, b_ld)).data):
        y = f()
        torch.manual_seed(3)
        g = torch.randn_like(y)
        (ga,) = torch.autograd.grad(y, a, g, create_graph=True)
        res.append(torch.autograd.grad((ga * u).sum(), (a, b)))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])


def test_banded_registrations_pass_opcheck_and_compile(gpu):
    a, b, band = band_pair(gpu, n=20, a_lu=2, a_ld=1, b_lu=1, b_ld=3)
    ad, bd = a.detach(), b.detach()
    tests = ("test_schema", "test_faketensor", "test_autograd_registration")
    for mode in (0, 1, 3):
        torch.library.opcheck(torch.ops.genbmm_amd.banded_fwd.default, (ad, bd) + band + (mode,), test_utils=tests)
        out, aux = torch.ops.genbmm_amd.banded_fwd(ad, bd, *band, mode)
        torch.library.opcheck(torch.ops.genbmm_amd.banded_bwd.default,
                              (ad, bd, out, aux, torch.randn_like(out)) + band + (mode,), test_utils=tests)

    def chain(x, y):
        z = ops.banded_multiply_log(x, 2, 1, y, 1, 3)      # band (5, 2)
        w = ops.banded_multiply(z, 5, 2, y, 1, 3)          # band (8, 3)
        return (w * w).sum() + ops.banded_multiply_max(x, 2, 1, y, 1, 3).sum()

    want = chain(a, b)
    wa, wb = torch.autograd.grad(want, (a, b))
    got = torch.compile(chain, backend="aot_eager", fullgraph=True)(a, b)
    ga, gb = torch.autograd.grad(got, (a, b))
    assert torch.equal(got, want) and torch.equal(ga, wa) and torch.equal(gb, wb)
