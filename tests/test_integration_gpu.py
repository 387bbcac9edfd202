"""The calling patterns of the library's main user (PyTorch-Struct's fast semirings):
leading dimensions flattened to one batch, `logbmm` / `maxbmm` combined in a log-depth
tree over a chain, and `b.multiply_log(a.transpose())` on banded operands.  Checked
against float64 dynamic programs written out sequentially."""
import math

import pytest
import torch

import genbmm_amd as genbmm
from genbmm_amd.sparse import BandedMatrix, banddiag

pytestmark = pytest.mark.gpu


def struct_matmul(op, a, b):
    """(..., M, K) x (..., K, N) the way the fast semirings call the library."""
    a2 = a.contiguous().view(-1, a.shape[-2], a.shape[-1])
    b2 = b.contiguous().view(-1, b.shape[-2], b.shape[-1])
    return op(a2, b2).view(a.shape[:-1] + (b.shape[-1],))


def chain_tree(op, pots):
    """pots (batch, N, C, C), N a power of two: combine neighbours pairwise, log2 N rounds."""
    cur = pots
    while cur.shape[1] > 1:
        cur = struct_matmul(op, cur[:, 0::2], cur[:, 1::2])
    return cur[:, 0]


@pytest.mark.parametrize("batch,N,C", [(3, 8, 5), (2, 32, 33), (4, 16, 128)])
def test_linear_chain_partition_and_marginals(gpu, batch, N, C):
    torch.manual_seed(N + C)
    pots = torch.randn(batch, N, C, C)
    x = pots.to(gpu).requires_grad_(True)
    z = chain_tree(genbmm.logbmm, x).logsumexp((-2, -1))
    # sequential forward algorithm in float64
    alpha = pots[:, 0].double()
    for t in range(1, N):
        alpha = (alpha.unsqueeze(-1) + pots[:, t].double().unsqueeze(-3)).logsumexp(-2)
    want = alpha.logsumexp((-2, -1))
    # log2(N) levels of logbmm and one logsumexp, each good to an ulp of its value
    tol = (math.log2(N) + 1) * float(torch.finfo(torch.float32).eps) * float(want.abs().max())
    assert torch.allclose(z.detach().cpu().double(), want, rtol=0, atol=tol)
    # d logZ / d potentials = edge marginals: each position's sum to one
    (marg,) = torch.autograd.grad(z.sum(), x)
    assert torch.allclose(marg.sum((-2, -1)).cpu(), torch.ones(batch, N), atol=1e-4)
    assert float(marg.min()) >= 0.0


def test_linear_chain_viterbi(gpu):
    torch.manual_seed(1)
    batch, N, C = 3, 16, 9
    pots = torch.round(torch.randn(batch, N, C, C) * 8) / 8
    x = pots.to(gpu).requires_grad_(True)
    best = chain_tree(genbmm.maxbmm, x).amax((-2, -1))
    alpha = pots[:, 0]
    for t in range(1, N):
        alpha = (alpha.unsqueeze(-1) + pots[:, t].unsqueeze(-3)).amax(-2)
    assert torch.equal(best.detach().cpu(), alpha.amax((-2, -1)))     # exact on the 1/8 grid
    # the gradient marks one edge per position on a best path; its score is the maximum
    (path,) = torch.autograd.grad(best.sum(), x)
    assert torch.equal(path.sum((-2, -1)).cpu(), torch.ones(batch, N))
    assert torch.equal((path.cpu() * pots).sum((1, 2, 3)), alpha.amax((-2, -1)))


def test_five_dimensional_operands(gpu):
    torch.manual_seed(2)
    a, b = torch.randn(2, 3, 4, 17, 9), torch.randn(2, 3, 4, 9, 21)
    got = struct_matmul(genbmm.logbmm, a.to(gpu), b.to(gpu))
    want = (a.double().unsqueeze(-1) + b.double().unsqueeze(-3)).logsumexp(-2)
    assert got.shape == (2, 3, 4, 17, 21)
    assert torch.allclose(got.cpu().double(), want, rtol=1e-5, atol=1e-5)
    # the same operands handed over as they are: leading dimensions are flattened inside
    direct = genbmm.logbmm(a.to(gpu), b.to(gpu))
    assert torch.equal(direct, got)
    # and a transposed view is made contiguous inside (the reference raises here)
    at = a.to(gpu).transpose(-1, -2).contiguous()
    assert torch.equal(genbmm.logbmm(at.transpose(-1, -2), b.to(gpu)), got)


@pytest.mark.parametrize("n,lu,ld", [(24, 2, 3), (70, 5, 1)])
def test_banded_semiring_matmul_pattern(gpu, n, lu, ld):
    """LogSemiring.matmul on banded operands: b.multiply_log(a.transpose())."""
    torch.manual_seed(n)
    da, db = torch.randn(2, n, n), torch.randn(2, n, n)
    a = BandedMatrix(banddiag(da, lu, ld, fill=-1e9)[0].to(gpu), lu, ld, fill=-1e9)
    b = BandedMatrix(banddiag(db, ld, lu, fill=-1e9)[0].to(gpu), ld, lu, fill=-1e9)
    got = b.multiply_log(a.transpose())
    # dense: Dense(a^T)^T (x) Dense(b) = Dense(a) (x) Dense(b) in the log semiring
    A, Bd = a.to_dense().double().cpu(), b.to_dense().double().cpu()
    want = (A.unsqueeze(-1) + Bd.unsqueeze(-3)).logsumexp(-2)
    dense = got.to_dense().double().cpu()
    r = torch.arange(n).unsqueeze(1)
    c = torch.arange(n).unsqueeze(0)
    inside = ((r - c) <= got.ld) & ((c - r) <= got.lu)
    assert torch.allclose(dense[:, inside], want[:, inside], rtol=1e-5, atol=1e-5)
    assert math.isfinite(float(dense[:, inside].abs().max()))
