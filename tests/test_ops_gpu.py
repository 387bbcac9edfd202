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


def test_registrations_pass_opcheck(gpu):
    a, b = pair(gpu, 2, 9, 12, 7)
    ad, bd = a.detach(), b.detach()
    tests = ("test_schema", "test_faketensor", "test_autograd_registration")
    torch.library.opcheck(torch.ops.genbmm_amd.logbmm_fwd.default, (ad, bd), test_utils=tests)
    torch.library.opcheck(torch.ops.genbmm_amd.maxbmm_fwd.default, (ad, bd), test_utils=tests)
    torch.library.opcheck(torch.ops.genbmm_amd.prodmaxbmm_fwd.default, (ad, bd), test_utils=tests)
    torch.library.opcheck(torch.ops.genbmm_amd.samplebmm_fwd.default, (ad, bd, 5, 0), test_utils=tests)
    out, idx = torch.ops.genbmm_amd.maxbmm_fwd(ad, bd)
    torch.library.opcheck(torch.ops.genbmm_amd.argmax_bwd.default, (idx, torch.randn_like(out), 12), test_utils=tests)


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
