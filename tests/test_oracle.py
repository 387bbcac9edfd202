"""Pins the CPU oracle (oracle/) - no GPU involved.

The reference stores no golden vectors for this path, so each oracle function is
pinned against something independent of its own formula:
  * Philox4x32-10: the Random123 known-answer vectors and a second, pure-Python
    implementation;
  * dense log/max/prod-max: torch's broadcast formulation (README.md:23-66) in
    float64 / bit-exact fp32, brute-force Python loops, special cases (K=1,
    constant inputs, masked rows);
  * gradients: torch autograd through the broadcast formulation (first and second
    order, test_cuda.py:22-42), row-sum invariants;
  * banded: dense torch.bmm / logsumexp / max identities of test_sparse.py and
    autograd through them.
"""
import math
import os

import numpy as np
import pytest
import torch

import oracle
from genbmm_amd.sparse import BandedMatrix, banddiag

torch.manual_seed(0)


# ------------------------------------------------------------------- Philox
KAT = [
    ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
    ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
     (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
]


@pytest.mark.parametrize("ctr,key,want", KAT)
def test_philox_known_answers(ctr, key, want):
    assert oracle.philox4x32_10(ctr, key) == want
    assert oracle.philox4x32_10_py(ctr, key) == want


def test_philox_uniform_mapping():
    seed, offset = 0x1234_5678_9ABC_DEF0, 0x0FED_CBA9_8765_4321
    first = (1 << 34) - 6  # crosses the 32-bit boundary of the block index (cell >> 2)
    u = oracle.philox_uniform(first, 12, seed, offset)
    for e in range(12):
        i = first + e
        blk = i >> 2                       # four consecutive cells share one Philox block
        x = oracle.philox4x32_10_py((blk & 0xFFFFFFFF, blk >> 32, offset & 0xFFFFFFFF, offset >> 32),
                                    (seed & 0xFFFFFFFF, seed >> 32))
        assert float(u[e]) == (x[i & 3] >> 8) / 16777216.0
    big = oracle.philox_uniform(0, 200000, 1234, 0)
    assert 0.0 <= float(big.min()) and float(big.max()) < 1.0
    assert abs(float(big.mean()) - 0.5) < 0.005
    hist = torch.histc(big, bins=16, min=0, max=1)
    chi2 = float(((hist - 12500) ** 2 / 12500).sum())
    assert chi2 < 50  # 15 dof, 1e-5 tail is 44.3... generous


# ------------------------------------------------------------- dense forward
def _rand(*shape):
    return torch.randn(*shape)


def test_seq_logbmm_fwd_matches_broadcast64():
    a, b = _rand(3, 7, 9).double(), _rand(3, 9, 5).double()
    out, mx = oracle.seq_logbmm_fwd(a, b, dtype=np.float64)
    want = oracle.logbmm_broadcast(a, b)
    assert torch.allclose(out, want, rtol=1e-13, atol=1e-13)
    assert torch.equal(mx, oracle.maxbmm_broadcast(a, b)[0])
    out32, _ = oracle.seq_logbmm_fwd(a, b)
    assert torch.allclose(out32.double(), want, rtol=1e-6, atol=1e-6)


def test_seq_logbmm_fwd_special_cases():
    a, b = _rand(2, 4, 1).double(), _rand(2, 1, 6).double()
    out, _ = oracle.seq_logbmm_fwd(a, b, dtype=np.float64)
    assert torch.allclose(out, a + b, rtol=0, atol=1e-15)  # K = 1
    a, b = torch.full((1, 3, 8), 0.25).double(), torch.full((1, 8, 2), -1.5).double()
    out, _ = oracle.seq_logbmm_fwd(a, b, dtype=np.float64)
    assert torch.allclose(out, torch.full((1, 3, 2), -1.25 + math.log(8)).double(), atol=1e-14)
    # a masked column of b (-inf) drops out; a fully masked row gives -inf
    a, b = _rand(1, 3, 4).double(), _rand(1, 4, 2).double()
    b[0, 1, :] = -math.inf
    out, _ = oracle.seq_logbmm_fwd(a, b, dtype=np.float64)
    keep = [0, 2, 3]
    assert torch.allclose(out, oracle.logbmm_broadcast(a[:, :, keep], b[:, keep, :]), atol=1e-14)
    a[0, 0, :] = -math.inf
    out, _ = oracle.seq_logbmm_fwd(a, b, dtype=np.float64)
    assert torch.isinf(out[0, 0]).all() and (out[0, 0] < 0).all()
    # the -1e9 floor: terms below it vanish (matmul_cuda_kernel.cu:31)
    a, b = torch.full((1, 1, 2), -2e9).double(), torch.zeros(1, 2, 1).double()
    out, mx = oracle.seq_logbmm_fwd(a, b, dtype=np.float64)
    assert float(mx) == -1e9 and float(out) == -math.inf


def _grid(*shape):
    return torch.round(torch.randn(*shape) * 8) / 8


def _brute_max(a, b, prod):
    B, M, K = a.shape
    N = b.shape[2]
    val = torch.empty(B, M, N)
    idx = torch.empty(B, M, N, dtype=torch.int32)
    for n in range(B):
        for r in range(M):
            for c in range(N):
                m, ind = np.float32(-1e9), -1
                for i in range(K):
                    x, y = np.float32(a[n, r, i]), np.float32(b[n, i, c])
                    v = np.float32(x * y) if prod else np.float32(x + y)
                    if v > m:
                        m, ind = v, i
                val[n, r, c], idx[n, r, c] = float(m), ind
    return val, idx


@pytest.mark.parametrize("prod", [False, True])
def test_seq_maxbmm_fwd_bit_exact(prod):
    a, b = _grid(4, 9, 17), _grid(4, 17, 6)  # 1/8 grid: many exact ties
    val, idx = oracle.seq_maxbmm_fwd(a, b, prod)
    tv, ti = (oracle.prodmaxbmm_broadcast if prod else oracle.maxbmm_broadcast)(a, b)
    assert torch.equal(val, tv) and torch.equal(idx.long(), ti)
    s = (a.unsqueeze(-1) * b.unsqueeze(-3)) if prod else (a.unsqueeze(-1) + b.unsqueeze(-3))
    assert int(((s == tv.unsqueeze(-2)).sum(-2) > 1).sum()) > 0  # ties really occur
    bv, bi = _brute_max(a[:2, :3], b[:2, :, :3], prod)
    assert torch.equal(val[:2, :3, :3], bv) and torch.equal(idx[:2, :3, :3], bi)


def test_seq_maxbmm_floor_and_empty():
    a, b = torch.full((1, 2, 3), -2e9), torch.zeros(1, 3, 2)
    val, idx = oracle.seq_maxbmm_fwd(a, b)
    assert (val == -1e9).all() and (idx == -1).all()


# ----------------------------------------------------------- dense backward
def test_seq_logbmm_bwd_matches_autograd64():
    a, b, g = _rand(2, 6, 8), _rand(2, 8, 5), _rand(2, 6, 5)
    ga, gb = oracle.seq_logbmm_bwd(a.double(), b.double(), g.double(), dtype=np.float64)
    _, wa, wb = oracle.logbmm_grads64(a, b, g)
    assert torch.allclose(ga, wa, rtol=1e-12, atol=1e-12)
    assert torch.allclose(gb, wb, rtol=1e-12, atol=1e-12)
    # softmax weights sum to one over k
    assert torch.allclose(ga.sum(-1), g.double().sum(-1), atol=1e-12)
    assert torch.allclose(gb.sum(-2), g.double().sum(-2), atol=1e-12)


def test_seq_logbmm_bwdbwd_matches_autograd64():
    a, b, g, u = _rand(2, 4, 5), _rand(2, 5, 3), _rand(2, 4, 3), _rand(2, 4, 5)
    got = oracle.seq_logbmm_bwdbwd(a.double(), b.double(), g.double(), u.double(), dtype=np.float64)
    want = oracle.logbmm_second_order64(a, b, g, u, None)
    for x, y in zip(got, want):
        assert torch.allclose(x, y, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("prod", [False, True])
def test_seq_argmax_bwd_matches_autograd(prod):
    if prod:
        a, b = (torch.randint(1, 9, (3, 7, 11)) / 8.0), (torch.randint(1, 9, (3, 11, 5)) / 8.0)
    else:
        a, b = _grid(3, 7, 11), _grid(3, 11, 5)
    g = _grid(3, 7, 5).clamp(-4, 4)
    _, idx = oracle.seq_maxbmm_fwd(a, b, prod)
    ga, gb = oracle.seq_argmax_bwd(a if prod else a.shape[2], b, idx, g, prod)
    ar, br = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
    val = (oracle.prodmaxbmm_broadcast if prod else oracle.maxbmm_broadcast)(ar, br)[0]
    wa, wb = torch.autograd.grad(val, (ar, br), g)
    # dyadic values with small magnitude: every partial sum is exact, so any order agrees
    assert torch.equal(ga, wa) and torch.equal(gb, wb)


def test_seq_prodmax_bwd_general_values_close():
    a, b = 1 - torch.rand(2, 6, 9), 1 - torch.rand(2, 9, 4)
    g = _rand(2, 6, 4)
    _, idx = oracle.seq_maxbmm_fwd(a, b, True)
    ga, gb = oracle.seq_argmax_bwd(a, b, idx, g, True)
    ar, br = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
    wa, wb = torch.autograd.grad(oracle.prodmaxbmm_broadcast(ar, br)[0], (ar, br), g)
    assert torch.allclose(ga, wa, rtol=1e-5, atol=1e-6) and torch.allclose(gb, wb, rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------- sample
def test_seq_sample_matches_cdf_rule_and_distribution():
    a, b = 2 * _rand(1, 2, 6), 2 * _rand(1, 6, 2)
    draws = 20000
    A, Bm = a.expand(draws, -1, -1).contiguous(), b.expand(draws, -1, -1).contiguous()
    u = oracle.philox_uniform(0, draws * 4, 99, 0).view(draws, 2, 2)
    out, idx = oracle.seq_samplebmm_fwd(A.double(), Bm.double(), u.double(), dtype=np.float64)
    assert torch.allclose(out, oracle.logbmm_broadcast(A.double(), Bm.double()), atol=1e-12)
    cdf = oracle.sample_cdf64(A, Bm)
    assert torch.equal(idx, oracle.sample_index_from_cdf(cdf, u))
    p = torch.softmax(a.double().unsqueeze(-1) + b.double().unsqueeze(-3), -2)[0]  # (M,K,N)
    for m in range(2):
        for n in range(2):
            cnt = torch.bincount(idx[:, m, n].long(), minlength=6).double()
            exp = p[m, :, n] * draws
            keep = exp >= 5
            chi2 = float((((cnt - exp) ** 2) / exp)[keep].sum())
            assert chi2 < 40, (m, n, chi2)
    # r = 0 never brackets: index stays 0 (reference :113 with total = 0)
    _, idx0 = oracle.seq_samplebmm_fwd(a, b, torch.zeros(1, 2, 2))
    assert (idx0 == 0).all()


# ------------------------------------------------------------------- banded
BANDS = [(5, 1, 1, 2, 0), (6, 2, 1, 1, 3), (4, 3, 3, 3, 3), (7, 0, 2, 2, 0), (3, 4, 5, 5, 4)]


def _band_pair(n, a_lu, a_ld, b_lu, b_ld, batch=2, grid=False):
    mk = _grid if grid else _rand
    a = oracle.band_from_dense(mk(batch, n, n), a_lu, a_ld)
    b = oracle.band_from_dense(mk(batch, n, n), b_lu, b_ld)
    return a, b


def test_band_layout_matches_host_banddiag():
    for n, lu, ld, _, _ in BANDS:
        x = _rand(2, n, n)
        assert torch.equal(oracle.band_from_dense(x, lu, ld), banddiag(x, lu, ld)[0])
        band = oracle.band_from_dense(x, lu, ld)
        assert torch.equal(oracle.band_to_dense(band, lu, ld, -7.0), BandedMatrix(band, lu, ld, -7.0).to_dense())
        assert torch.equal(oracle.band_transpose_indexed(band, lu, ld), oracle.band_transpose(band, lu, ld))


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", BANDS)
@pytest.mark.parametrize("mode", [0, 1, 3])
def test_seq_band_fwd_matches_dense_identity(n, a_lu, a_ld, b_lu, b_ld, mode):
    a, b = _band_pair(n, a_lu, a_ld, b_lu, b_ld)
    out, idx, _ = oracle.seq_band_fwd(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, mode, dtype=np.float64)
    want, mask = oracle.band_product_dense(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, mode)
    assert torch.allclose(out[:, mask], want[:, mask], rtol=1e-12, atol=1e-12)
    assert (out[:, ~mask] == 0).all()  # cells outside the matrix keep the zero fill


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", BANDS)
def test_seq_band_sample_matches_dense_sample_rule(n, a_lu, a_ld, b_lu, b_ld):
    """The banded sample product has no reference function (the band kernel stops at modes 0, 1,
    3); its oracle is pinned through the dense identity of test_sparse.py:181-195 and the dense
    sampling oracle (itself pinned above): sampling Dense(b)^T (x) Dense(a) with -1e9 outside the
    bands picks, for result cell (r, c), a dense row p of a's column c, i.e. k = p - c + a_lu."""
    a, b = _band_pair(n, a_lu, a_ld, b_lu, b_ld)
    a, b = 2 * a.double(), 2 * b.double()
    lu, ld = a_lu + b_ld, a_ld + b_lu
    W = lu + ld + 1
    u = oracle.philox_uniform(0, 2 * n * W, 7, 3).view(2, n, W).double().clamp(min=1e-3)
    out, idx = oracle.seq_band_sample_fwd(a, a_lu, a_ld, b, b_lu, b_ld, u, dtype=np.float64)
    want, mask = oracle.band_product_dense(a, a_lu, a_ld, b, b_lu, b_ld, 0)
    assert torch.allclose(out[:, mask], want[:, mask], rtol=1e-12, atol=1e-12)
    assert (out[:, ~mask] == 0).all() and (idx[:, ~mask] == 0).all()
    X = oracle.band_to_dense(a, a_lu, a_ld, -1e9)
    Y = oracle.band_to_dense(b, b_lu, b_ld, -1e9)
    ud = oracle.band_to_dense(u, lu, ld, 0.5)                 # uniforms at their dense cells (r, c)
    _, p = oracle.seq_samplebmm_fwd(Y.transpose(-2, -1).contiguous(), X, ud, dtype=np.float64)
    k_dense = p - torch.arange(n).view(1, 1, n) + a_lu            # (B, r, c)
    k_band = oracle.band_from_dense(k_dense.double(), lu, ld).long()
    assert torch.equal(idx.long()[:, mask], k_band[:, mask])
    # and the float64 CDF rule evaluated by index arithmetic agrees
    cdf, valid = oracle.band_sample_cdf64(a, a_lu, a_ld, b, b_lu, b_ld)
    assert torch.equal(idx, oracle.band_sample_index_from_cdf(cdf, valid, u))
    # the terms tensor itself: its log-sum-exp is the product
    v, _ = oracle.band_terms64(a, a_lu, a_ld, b, b_lu, b_ld)
    assert torch.allclose(v.logsumexp(-1)[:, mask], want[:, mask], rtol=1e-12, atol=1e-12)


def test_seq_band_sample_distribution_and_defaults():
    n, a_lu, a_ld, b_lu, b_ld = 4, 1, 2, 2, 1
    a, b = _band_pair(n, a_lu, a_ld, b_lu, b_ld, batch=1)
    a, b = 2 * a.double(), 2 * b.double()
    W = a.shape[2] + b.shape[2] - 1
    draws = 20000
    A, Bm = a.expand(draws, -1, -1).contiguous(), b.expand(draws, -1, -1).contiguous()
    u = oracle.philox_uniform(0, draws * n * W, 5, 1).view(draws, n, W).double()
    _, idx = oracle.seq_band_sample_fwd(A, a_lu, a_ld, Bm, b_lu, b_ld, u, dtype=np.float64)
    cdf, valid = oracle.band_sample_cdf64(a, a_lu, a_ld, b, b_lu, b_ld)
    pr = torch.diff(cdf[0], dim=-1, prepend=torch.zeros(n, W, 1, dtype=torch.float64))
    for i in range(n):
        for j in range(W):
            if not valid[i, j].any():
                assert (idx[:, i, j] == 0).all()
                continue
            cnt = torch.bincount(idx[:, i, j].long(), minlength=a.shape[2]).double()
            assert (cnt[~valid[i, j]] == 0).all()              # only terms of the cell are drawn
            exp = pr[i, j] * draws
            keep = exp >= 5
            assert float((((cnt - exp) ** 2) / exp)[keep].sum()) < 45, (i, j)
    # r = 0 never brackets: every cell keeps its first term
    _, idx0 = oracle.seq_band_sample_fwd(a, a_lu, a_ld, b, b_lu, b_ld, torch.zeros(1, n, W), dtype=np.float64)
    first = valid.to(torch.int8).argmax(-1)
    assert torch.equal(idx0[0].long(), torch.where(valid.any(-1), first, torch.zeros_like(first)))


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", BANDS)
def test_band_closed_forms_by_index_arithmetic_match_the_dense_identity(n, a_lu, a_ld, b_lu, b_ld):
    """band_product64 / band_max_first (used on the device for full-size checks) against the
    dense identities of test_sparse.py:141-142, 181-195 and the sequential kernel restatement."""
    a, b = _band_pair(n, a_lu, a_ld, b_lu, b_ld, grid=True)
    for mode in (3, 0):
        want, mask = oracle.band_product_dense(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld, mode)
        got = oracle.band_product64(a, a_lu, a_ld, b, b_lu, b_ld, mode)
        assert torch.allclose(got[:, mask], want[:, mask], rtol=1e-12, atol=1e-12)
        assert (got[:, ~mask] == 0).all()
    sv, si, _ = oracle.seq_band_fwd(a, a_lu, a_ld, b, b_lu, b_ld, 1)
    mv, mi = oracle.band_max_first(a, a_lu, a_ld, b, b_lu, b_ld)
    assert torch.equal(mv, sv) and torch.equal(mi, si)          # ties present on the 1/8 grid


def _dense_band_fn(a_lu, a_ld, b_lu, b_ld, mode):
    fill = 0.0 if mode == 3 else -1e9

    def fn(a, b):
        X = BandedMatrix(a, a_lu, a_ld, fill).to_dense()
        Y = BandedMatrix(b, b_lu, b_ld, fill).to_dense()
        if mode == 3:
            D = torch.bmm(Y.transpose(-2, -1), X)
        else:
            S = Y.transpose(-2, -1).unsqueeze(-1) + X.unsqueeze(-3)
            D = S.logsumexp(-2) if mode == 0 else S.max(-2).values
        return banddiag(D, a_lu + b_ld, a_ld + b_lu)[0]

    return fn


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", BANDS)
@pytest.mark.parametrize("mode", [0, 1, 3])
def test_seq_band_bwd_matches_autograd(n, a_lu, a_ld, b_lu, b_ld, mode):
    a, b = _band_pair(n, a_lu, a_ld, b_lu, b_ld)
    a, b = a.double(), b.double()
    W = a.shape[2] + b.shape[2] - 1
    g = _rand(2, n, W).double()
    ga, gb = oracle.seq_band_bwd(a, a_lu, a_ld, b, b_lu, b_ld, g, mode, dtype=np.float64)
    ar, br = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
    out = _dense_band_fn(a_lu, a_ld, b_lu, b_ld, mode)(ar, br)
    wa, wb = torch.autograd.grad(out, (ar, br), g)
    # band cells outside the matrix: the dense form never reads them (grad 0), and
    # the reference kernel leaves its zero fill there
    assert torch.allclose(ga, wa, rtol=1e-10, atol=1e-12)
    assert torch.allclose(gb, wb, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("n,a_lu,a_ld,b_lu,b_ld", BANDS[:3])
def test_seq_band_bwdbwd_matches_autograd(n, a_lu, a_ld, b_lu, b_ld):
    a, b = _band_pair(n, a_lu, a_ld, b_lu, b_ld)
    a, b = a.double(), b.double()
    W = a.shape[2] + b.shape[2] - 1
    g, u = _rand(2, n, W).double(), _rand(*a.shape).double()
    got = oracle.seq_band_bwdbwd(a, a_lu, a_ld, b, b_lu, b_ld, g, u, dtype=np.float64)
    ar, br, gr = (t.clone().requires_grad_(True) for t in (a, b, g))
    out = _dense_band_fn(a_lu, a_ld, b_lu, b_ld, 0)(ar, br)
    (ga,) = torch.autograd.grad(out, (ar,), gr, create_graph=True)
    want = torch.autograd.grad(ga, (ar, br, gr), u)
    for x, y in zip(got, want):
        assert torch.allclose(x, y, rtol=1e-9, atol=1e-11)


# ------------------------------------------------------------- golden fixtures
# Vectors written by the reference's own CPU code (the *_simple Python loops of
# genbmm/sparse.py:268-401, run by tests/golden/make_band_struct_fixtures.py).
@pytest.mark.parametrize("case", range(4))
def test_band_products_match_reference_cpu_loops(case):
    import os

    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "band_struct.npz"),
                allow_pickle=False)
    p = "c%d_" % case
    B, n, lu, ld, olu, old = (int(v) for v in z[p + "meta"])
    a, b = torch.from_numpy(z[p + "zband"]), torch.from_numpy(z[p + "zoband"])
    for mode, name in ((3, "multiply_simple"), (0, "multiply_log_simple"), (1, "multiply_max_simple")):
        got = oracle.seq_band_fwd(a, lu, ld, b, olu, old, mode)[0]
        assert [lu + old, ld + olu] == [int(v) for v in z[p + name + "_luld"]]
        assert torch.equal(got, torch.from_numpy(z[p + name])), name   # same loop order, fp32: bit for bit
    # multiply_back_simple returns the first operand's gradient in transposed band form
    g = torch.from_numpy(z[p + "grad_out"])
    ga, _ = oracle.seq_band_bwd(a, lu, ld, b, olu, old, g, 3)
    want = torch.from_numpy(z[p + "multiply_back_simple"])
    assert [ld, lu] == [int(v) for v in z[p + "multiply_back_simple_luld"]]
    assert torch.allclose(oracle.band_transpose(ga, lu, ld), want, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("case", range(4))
def test_band_relabel_and_op_match_reference_vectors(case):
    """oracle.band_relabel / band_op / band_transpose_indexed / band_to_dense against the
    outputs of the reference's own BandedMatrix methods (tests/golden/band_struct.npz)."""
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "band_struct.npz"), allow_pickle=False)
    p = "c%d_" % case
    B, n, lu, ld, olu, old = (int(v) for v in z[p + "meta"])
    fill = float(z[p + "fill"])
    band, oband = torch.from_numpy(z[p + "band"]), torch.from_numpy(z[p + "oband"])
    W = lu + ld + 1

    def same(name, got):
        assert torch.equal(got, torch.from_numpy(z[p + name])), name

    same("band_shift_p1", oracle.band_relabel(band, 0, 1, W, fill))
    same("band_shift_m2", oracle.band_relabel(band, 0, -2, W, fill))
    same("band_pad_2", oracle.band_relabel(band, 0, -2, W + 4, fill))
    same("band_unshift", oracle.band_relabel(band, 0, -1, W, fill))
    same("col_shift_p1", oracle.band_relabel(band, 1, 0, W, fill))
    same("col_shift_m2", oracle.band_relabel(band, -2, 0, W, fill))
    same("col_unshift", oracle.band_relabel(band, -1, 0, W, fill))
    same("expand", oracle.band_relabel(band, 0, -2, W + 3, fill))
    got, glu, gld = oracle.band_op(band, lu, ld, oband, olu, old, np.add, 0.0)
    assert [glu, gld] == [int(v) for v in z[p + "op_add_luld"]]
    same("op_add", got)
    same("op_max", oracle.band_op(band, lu, ld, oband, olu, old, np.maximum, -1e9)[0])
    same("transpose", oracle.band_transpose_indexed(band, lu, ld))
    same("to_dense", oracle.band_to_dense(band, lu, ld, fill))
