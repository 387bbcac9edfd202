"""float16 / bfloat16 tensors through the dense entry points (`*_f16`, `*_bf16`): the kernels
are the float kernels compiled for that element type - loads widen, arithmetic and workspaces
are fp32, stores round to nearest - so the contract tested here is exact: every result equals
what the float entry point returns on the widened tensors, rounded once (indices identical),
for every kernel family a shape can take.  On top of that the results are compared with the
float64 closed forms / the sequential oracle at the tolerance of one rounding of the output
type.  (The reference computes in scalar_t = Half, matmul_cuda_kernel.cu:489; it has no test
for it.)"""
import pytest
import torch

import oracle
import genbmm_amd as genbmm
from genbmm_amd import _lib

pytestmark = pytest.mark.gpu

TYPES = [(torch.float16, "_f16", 2.0 ** -11), (torch.bfloat16, "_bf16", 2.0 ** -8)]
# whole items (32^3 on the matrix cores, up to 64^3 in LDS), one 128 x 128 tile per item, tiled
# matrix-core shapes (full tiles, ragged, 256-wide tiles), vector-ALU shapes, odd alignments
SHAPES = [(3, 32, 32, 32), (2, 64, 64, 64), (3, 20, 33, 50), (5, 128, 128, 128), (3, 100, 96, 120),
          (2, 256, 128, 256), (2, 200, 77, 131), (2, 70, 50, 90), (1, 33, 17, 200), (2, 129, 513, 257),
          (8, 512, 256, 512)]
P = _lib.ptr


def lse64(a, b, chunk=2):
    """float64 logsumexp of the broadcast form (README.md:23-30 of the reference), in batch chunks."""
    outs = [oracle.logbmm_broadcast(a[i:i + chunk].double(), b[i:i + chunk].double())
            for i in range(0, a.shape[0], chunk)]
    return torch.cat(outs) if outs else a.new_zeros((0, a.shape[1], b.shape[2])).double()


def _operands(gpu, dt, B, M, K, N, scale=2.0):
    a = (scale * torch.randn(B, M, K, device=gpu)).to(dt)
    b = (scale * torch.randn(B, K, N, device=gpu)).to(dt)
    g = torch.randn(B, M, N, device=gpu).to(dt)
    return a, b, g


@pytest.mark.parametrize("dt,suffix,eps", TYPES)
@pytest.mark.parametrize("path", [genbmm.genmul.PATH_AUTO, genbmm.genmul.PATH_EXACT, genbmm.genmul.PATH_VALU,
                                  genbmm.genmul.PATH_FACTORS])
def test_logbmm_half_equals_float_kernels_rounded(gpu, dt, suffix, eps, path):
    lib = _lib.load()
    torch.manual_seed(3)
    for B, M, K, N in SHAPES:
        a, b, g = _operands(gpu, dt, B, M, K, N)
        a32, b32, g32 = a.float(), b.float(), g.float()
        n = lib.genbmm_logbmm_stats_size_path(B, M, K, N, path)
        st, st32 = torch.empty(n, device=gpu), torch.empty(n, device=gpu)
        out, out32 = torch.empty(B, M, N, device=gpu, dtype=dt), torch.empty(B, M, N, device=gpu)
        s = _lib.stream_of(a)
        assert getattr(lib, "genbmm_logbmm_fwd_path" + suffix)(P(a), P(b), P(out), P(st), B, M, K, N, path, s) == 0
        assert lib.genbmm_logbmm_fwd_path(P(a32), P(b32), P(out32), P(st32), B, M, K, N, path, s) == 0
        assert torch.equal(out, out32.to(dt)), (B, M, K, N)
        if B * M * K * N <= 40_000_000:
            want = lse64(a32.cpu(), b32.cpu())
            # one rounding of the result (half an ulp: eps relative) on top of the fp32 kernel's own error
            err = (out.double().cpu() - want).abs()
            assert bool((err <= eps * want.abs() + 1e-5 * want.abs() + 1e-6).all()), (B, M, K, N, float(err.max()))
        # the backward reads `out` as stored (rounded): the float kernels get the same values
        ga, gb = torch.empty_like(a), torch.empty_like(b)
        ga32, gb32 = torch.empty_like(a32), torch.empty_like(b32)
        oh = out.float()
        assert getattr(lib, "genbmm_logbmm_bwd_path" + suffix)(P(a), P(b), P(out), P(g), P(st), P(ga), P(gb),
                                                              B, M, K, N, path, s) == 0
        assert lib.genbmm_logbmm_bwd_path(P(a32), P(b32), P(oh), P(g32), P(st32), P(ga32), P(gb32),
                                          B, M, K, N, path, s) == 0
        assert torch.equal(ga, ga32.to(dt)) and torch.equal(gb, gb32.to(dt)), (B, M, K, N)


def _odd_shapes(seed, count, kmax):
    """Extents on both sides of every tile, slab and vector boundary, odd row lengths (rows of a
    half tensor then start at any 2-byte address)."""
    import random
    rng = random.Random(seed)
    edge = [1, 2, 3, 7, 8, 9, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 130, 255, 257]
    out = []
    for _ in range(count):
        M = rng.choice(edge + [rng.randint(1, 300)])
        N = rng.choice(edge + [rng.randint(1, 300)])
        K = rng.choice([1, 2, 7, 8, 9, 15, 16, 17, 31, 33, 127, 128, 129, 255, 257, rng.randint(1, kmax)])
        B = rng.randint(1, 3)
        if B * M * K * N > 8_000_000:
            K = max(1, 8_000_000 // (B * M * N))
        out.append((B, M, K, N))
    return out


@pytest.mark.parametrize("dt,suffix,eps", TYPES)
def test_half_equals_float_kernels_on_many_shapes(gpu, dt, suffix, eps):
    """The bit-for-bit contract on sixty seeded shapes: logbmm forward and backward (default
    path), maxbmm and prodmaxbmm values, indices and gradients."""
    lib = _lib.load()
    torch.manual_seed(9)
    for B, M, K, N in _odd_shapes(17, 60, 600):
        a, b, g = _operands(gpu, dt, B, M, K, N)
        a32, b32, g32 = a.float(), b.float(), g.float()
        s = _lib.stream_of(a)
        n = lib.genbmm_logbmm_stats_size(B, M, K, N)
        st, st32 = torch.empty(n, device=gpu), torch.empty(n, device=gpu)
        out, out32 = torch.empty(B, M, N, device=gpu, dtype=dt), torch.empty(B, M, N, device=gpu)
        assert getattr(lib, "genbmm_logbmm_fwd" + suffix)(P(a), P(b), P(out), P(st), B, M, K, N, s) == 0
        assert lib.genbmm_logbmm_fwd(P(a32), P(b32), P(out32), P(st32), B, M, K, N, s) == 0
        assert torch.equal(out, out32.to(dt)), ("logbmm", B, M, K, N)
        ga, gb = torch.empty_like(a), torch.empty_like(b)
        ga32, gb32 = torch.empty_like(a32), torch.empty_like(b32)
        oh = out.float()
        assert getattr(lib, "genbmm_logbmm_bwd" + suffix)(P(a), P(b), P(out), P(g), P(st), P(ga), P(gb), B, M, K, N, s) == 0
        assert lib.genbmm_logbmm_bwd(P(a32), P(b32), P(oh), P(g32), P(st32), P(ga32), P(gb32), B, M, K, N, s) == 0
        assert torch.equal(ga, ga32.to(dt)) and torch.equal(gb, gb32.to(dt)), ("logbmm bwd", B, M, K, N)
        idx, idx32 = (torch.empty(B, M, N, device=gpu, dtype=torch.int32) for _ in range(2))
        fac, fac32 = (torch.empty(2, B, M, N, device=gpu) for _ in range(2))
        assert getattr(lib, "genbmm_maxbmm_fwd" + suffix)(P(a), P(b), P(out), P(idx), B, M, K, N, s) == 0
        assert lib.genbmm_maxbmm_fwd(P(a32), P(b32), P(out32), P(idx32), B, M, K, N, s) == 0
        assert torch.equal(out, out32.to(dt)) and torch.equal(idx, idx32), ("maxbmm", B, M, K, N)
        assert getattr(lib, "genbmm_argmax_bwd" + suffix)(P(idx), P(g), P(ga), P(gb), B, M, K, N, s) == 0
        assert lib.genbmm_argmax_bwd(P(idx32), P(g32), P(ga32), P(gb32), B, M, K, N, s) == 0
        assert torch.equal(ga, ga32.to(dt)) and torch.equal(gb, gb32.to(dt)), ("argmax bwd", B, M, K, N)
        assert getattr(lib, "genbmm_prodmaxbmm_fwd" + suffix)(P(a), P(b), P(out), P(idx), P(fac), B, M, K, N, s) == 0
        assert lib.genbmm_prodmaxbmm_fwd(P(a32), P(b32), P(out32), P(idx32), P(fac32), B, M, K, N, s) == 0
        assert torch.equal(out, out32.to(dt)) and torch.equal(idx, idx32) and torch.equal(fac, fac32), ("prodmax", B, M, K, N)
        assert getattr(lib, "genbmm_prodmax_bwd" + suffix)(P(None), P(None), P(idx), P(fac), P(g), P(ga), P(gb), B, M, K, N, s) == 0
        assert lib.genbmm_prodmax_bwd(P(None), P(None), P(idx32), P(fac32), P(g32), P(ga32), P(gb32), B, M, K, N, s) == 0
        assert torch.equal(ga, ga32.to(dt)) and torch.equal(gb, gb32.to(dt)), ("prodmax bwd", B, M, K, N)


@pytest.mark.parametrize("dt,suffix,eps", TYPES)
def test_logbmm_half_gradients_against_float64(gpu, dt, suffix, eps):
    """Through the autograd layer, against float64 autograd of the closed form on the same
    (half-valued) operands.  The weights exp(a + b - out) are formed with `out` as stored:
    its rounding (eps |out|) enters every gradient term as a relative error."""
    torch.manual_seed(4)
    for B, M, K, N in [(3, 32, 32, 32), (2, 50, 40, 70), (4, 128, 128, 128), (2, 256, 128, 256), (2, 130, 97, 150)]:
        a, b, g = _operands(gpu, dt, B, M, K, N, scale=1.0)
        want, wa, wb = oracle.logbmm_grads64(a.float().cpu(), b.float().cpu(), g.float().cpu())
        ad, bd = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
        out = genbmm.logbmm(ad, bd)
        assert out.dtype == dt
        ga, gb = torch.autograd.grad(out, (ad, bd), g)
        assert ga.dtype == dt and gb.dtype == dt
        omax = float(want.abs().max())
        for got, ref in ((ga, wa), (gb, wb)):
            scale = float(ref.abs().max())
            tol = (2.0 * eps * omax + 2.0 * eps) * scale + 1e-6
            assert float((got.double().cpu() - ref).abs().max()) <= tol, (B, M, K, N)


@pytest.mark.parametrize("dt,suffix,eps", TYPES)
@pytest.mark.parametrize("prod", [False, True])
def test_max_products_half_bit_exact(gpu, dt, suffix, eps, prod):
    """Values and indices equal the sequential oracle's on the widened operands (values
    rounded once: a + b and a * b of two half values are exact in fp32), and so do the
    gradients, whose ordered fp32 sums are rounded once."""
    torch.manual_seed(5)
    for B, M, K, N in [(3, 20, 33, 50), (2, 64, 64, 64), (2, 200, 77, 131), (1, 33, 300, 200), (2, 129, 513, 70)]:
        a, b, g = _operands(gpu, dt, B, M, K, N)
        g = (torch.round(g.float() * 8) / 8).to(dt)
        sv, si = oracle.seq_maxbmm_fwd(a.float().cpu(), b.float().cpu(), prod)
        ad, bd = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
        out = (genbmm.prodmaxbmm if prod else genbmm.maxbmm)(ad, bd)
        assert out.dtype == dt
        assert torch.equal(out.detach().cpu(), sv.to(dt)), (B, M, K, N)
        ga, gb = torch.autograd.grad(out, (ad, bd), g)
        wa, wb = oracle.seq_argmax_bwd(a.float().cpu() if prod else K, b.float().cpu(), si, g.float().cpu(), prod)
        assert torch.equal(ga.cpu(), wa.to(dt)) and torch.equal(gb.cpu(), wb.to(dt)), (B, M, K, N)
        # the gathering form of the product backward (no stored factors) agrees
        if prod:
            lib = _lib.load()
            idx = si.to(gpu).to(torch.int32)
            ga2, gb2 = torch.empty_like(a), torch.empty_like(b)
            assert getattr(lib, "genbmm_prodmax_bwd" + suffix)(P(a), P(b), P(idx), P(None), P(g), P(ga2), P(gb2),
                                                              B, M, K, N, _lib.stream_of(a)) == 0
            assert torch.equal(ga2, ga) and torch.equal(gb2, gb)


@pytest.mark.parametrize("dt,suffix,eps", TYPES)
def test_samplebmm_half(gpu, dt, suffix, eps):
    """Every index brackets its uniform in the float64 CDF of the (half-valued) operands;
    shapes that take the matrix-core sweep (1/S from the fp32 workspace) and shapes that walk
    exactly; out is the float result rounded once."""
    lib = _lib.load()
    torch.manual_seed(6)
    for B, M, K, N in [(3, 20, 33, 50), (5, 128, 128, 128), (2, 200, 77, 131), (2, 256, 512, 128), (1, 128, 1040, 160),
                       (2, 64, 300, 96)]:
        a, b, _ = _operands(gpu, dt, B, M, K, N)
        out = torch.empty(B, M, N, device=gpu, dtype=dt)
        idx = torch.empty(B, M, N, dtype=torch.int32, device=gpu)
        stats = torch.empty(lib.genbmm_samplebmm_stats_size(B, M, K, N), device=gpu)
        assert getattr(lib, "genbmm_samplebmm_fwd" + suffix)(P(a), P(b), P(out), P(idx), P(stats), 21, 4, B, M, K, N,
                                                            _lib.stream_of(a)) == 0
        a32, b32 = a.float().cpu(), b.float().cpu()
        want = lse64(a32, b32)
        err = (out.double().cpu() - want).abs()
        assert bool((err <= eps * want.abs() + 1e-5 * want.abs() + 1e-6).all()), (B, M, K, N)
        u = oracle.philox_uniform(0, B * M * N, 21, 4).view(B, M, N).double()
        cdf = oracle.sample_cdf64(a32, b32)
        got = idx.cpu().long()
        assert int(got.min()) >= 0 and int(got.max()) < K
        hi = torch.gather(cdf, 2, got.unsqueeze(2)).squeeze(2)
        lo = torch.where(got > 0, torch.gather(cdf, 2, (got - 1).clamp(min=0).unsqueeze(2)).squeeze(2),
                         torch.zeros_like(hi))
        tol = max(2e-5, 2.0 * K * 2.0 ** -24)
        assert bool(((lo - tol <= u) & (u <= hi + tol)).all()), (B, M, K, N)
        # through the autograd layer: one-hot gradient of the sampled term
        ad = a.clone().requires_grad_(True)
        s = genbmm.samplebmm(ad, b, (21, 4))
        (ga,) = torch.autograd.grad(s.sum(), ad)
        assert ga.dtype == dt and float(ga.float().sum()) == pytest.approx(B * M * N, rel=1e-2)


@pytest.mark.parametrize("dt,suffix,eps", TYPES)
def test_half_tensors_at_any_two_byte_address(gpu, dt, suffix, eps):
    """Operands, results and gradients that start one element past a 16-byte boundary (views
    into larger buffers): the same bits as from aligned tensors, on shapes of every family."""
    lib = _lib.load()
    torch.manual_seed(10)

    def shifted(t):   # the same values at an address that is 2 mod 16
        buf = torch.empty(t.numel() + 9, device=gpu, dtype=dt)
        v = buf[1:1 + t.numel()].view(t.shape)
        v.copy_(t)
        assert v.data_ptr() % 16 == 2
        return v

    for B, M, K, N in [(3, 32, 32, 32), (2, 40, 24, 36), (2, 128, 128, 128), (2, 100, 96, 120), (2, 256, 128, 256),
                       (1, 129, 77, 131)]:
        a, b, g = _operands(gpu, dt, B, M, K, N)
        s = _lib.stream_of(a)
        n = lib.genbmm_logbmm_stats_size(B, M, K, N)
        res = []
        for move in (lambda t: t, shifted):
            x, y, gg = move(a), move(b), move(g)
            st = torch.empty(n, device=gpu)
            out, ga, gb = move(torch.zeros(B, M, N, device=gpu, dtype=dt)), move(torch.zeros_like(a)), move(torch.zeros_like(b))
            assert getattr(lib, "genbmm_logbmm_fwd" + suffix)(P(x), P(y), P(out), P(st), B, M, K, N, s) == 0
            assert getattr(lib, "genbmm_logbmm_bwd" + suffix)(P(x), P(y), P(out), P(gg), P(st), P(ga), P(gb), B, M, K, N, s) == 0
            mo, idx = move(torch.zeros(B, M, N, device=gpu, dtype=dt)), torch.empty(B, M, N, device=gpu, dtype=torch.int32)
            assert getattr(lib, "genbmm_maxbmm_fwd" + suffix)(P(x), P(y), P(mo), P(idx), B, M, K, N, s) == 0
            ma, mb = move(torch.zeros_like(a)), move(torch.zeros_like(b))
            assert getattr(lib, "genbmm_argmax_bwd" + suffix)(P(idx), P(gg), P(ma), P(mb), B, M, K, N, s) == 0
            res.append([t.clone() for t in (out, ga, gb, mo, idx, ma, mb)])
        for u, v in zip(*res):
            assert torch.equal(u, v), (B, M, K, N)


def test_half_masks_and_empty(gpu):
    """-inf masks, rows without mass, the reference's -1e9 floor (which is -inf in
    binary16, as `scalar_t m = -1e9` is in the reference) and empty extents."""
    for dt in (torch.float16, torch.bfloat16):
        torch.manual_seed(8)
        a = torch.randn(2, 70, 40, device=gpu).to(dt)
        b = torch.randn(2, 40, 90, device=gpu).to(dt)
        a[:, ::3, ::5] = float("-inf")
        a[1, 5, :] = float("-inf")
        out = genbmm.logbmm(a, b)
        want = lse64(a.float().cpu(), b.float().cpu())
        assert bool(torch.isneginf(out[1, 5]).all())
        live = torch.isfinite(want)
        eps = 2.0 ** -11 if dt == torch.float16 else 2.0 ** -8
        assert bool(((out.double().cpu() - want).abs()[live] <= eps * want.abs()[live] + 1e-4).all())
        for shape in [(0, 3, 4, 5), (2, 0, 4, 5), (2, 3, 4, 0)]:
            B, M, K, N = shape
            z = genbmm.logbmm(torch.randn(B, M, K, device=gpu).to(dt), torch.randn(B, K, N, device=gpu).to(dt))
            assert z.shape == (B, M, N) and z.dtype == dt
        e = genbmm.maxbmm(torch.randn(2, 3, 0, device=gpu).to(dt), torch.randn(2, 0, 5, device=gpu).to(dt))
        floor = torch.full(e.shape, -1e9, device=gpu).to(dt)   # rounded to the type (-inf in binary16)
        assert torch.equal(e, floor)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_banded_products_on_half_bands(gpu, dt):
    """BandedMatrix widens half bands for the banded kernels and narrows the result: the float
    product of the widened bands, rounded once; gradients arrive in the half tensors."""
    from genbmm_amd.sparse import BandedMatrix, banddiag
    torch.manual_seed(11)
    n, (alu, ald, blu, bld) = 70, (5, 3, 2, 6)
    x = banddiag(torch.randn(2, n, n), alu, ald)[0].contiguous().to(gpu).to(dt)
    y = banddiag(torch.randn(2, n, n), blu, bld)[0].contiguous().to(gpu).to(dt)
    for name in ("multiply", "multiply_log", "multiply_max"):
        xh, yh = x.clone().requires_grad_(True), y.clone().requires_grad_(True)
        got = getattr(BandedMatrix(xh, alu, ald), name)(BandedMatrix(yh, blu, bld))
        want = getattr(BandedMatrix(x.float(), alu, ald), name)(BandedMatrix(y.float(), blu, bld))
        assert got.data.dtype == dt and (got.lu, got.ld) == (want.lu, want.ld)
        assert torch.equal(got.data, want.data.to(dt)), name
        ga, gb = torch.autograd.grad(got.data.float().sum(), (xh, yh))
        assert ga.dtype == dt and gb.dtype == dt and float(ga.float().abs().sum()) > 0


@pytest.mark.parametrize("dt,suffix,eps", TYPES)
@pytest.mark.parametrize("B,M,K,N", [(3, 20, 33, 50), (6, 128, 128, 128), (4, 100, 70, 130)])
def test_logbmm_second_order_half_equals_float_kernels_rounded(gpu, dt, suffix, eps, B, M, K, N):
    """genbmm_logbmm_bwdbwd_ws_f16 / _bf16 (exact passes for the small shape, matrix cores for the
    others): the float function on the widened tensors, rounded once - the gradient with respect
    to g stays unrounded in the workspace for the other two gradients."""
    lib = _lib.load()
    torch.manual_seed(B + M)
    a, b, g = _operands(gpu, dt, B, M, K, N, scale=1.0)
    ua, ub = torch.randn(B, M, K, device=gpu).to(dt), torch.randn(B, K, N, device=gpu).to(dt)
    s = _lib.stream_of(a)
    out = torch.empty(B, M, N, device=gpu, dtype=dt)
    st = torch.empty(lib.genbmm_logbmm_stats_size(B, M, K, N), device=gpu)
    assert getattr(lib, "genbmm_logbmm_fwd" + suffix)(P(a), P(b), P(out), P(st), B, M, K, N, s) == 0
    wide = [t.float() for t in (a, b, out, g, ua, ub)]
    nws = lib.genbmm_logbmm_bwdbwd_ws_size(B, M, K, N)
    for u_a, u_b, w_a, w_b in ((ua, ub, wide[4], wide[5]), (ua, None, wide[4], None), (None, ub, None, wide[5])):
        ws, ws32 = torch.empty(nws, device=gpu), torch.empty(nws, device=gpu)
        ga, gb, gg = torch.empty_like(a), torch.empty_like(b), torch.empty_like(g)
        ga32, gb32, gg32 = (torch.empty_like(t) for t in (wide[0], wide[1], wide[3]))
        assert getattr(lib, "genbmm_logbmm_bwdbwd_ws" + suffix)(P(a), P(b), P(out), P(g), P(u_a), P(u_b), P(ga), P(gb),
                                                               P(gg), P(ws), B, M, K, N, s) == 0
        assert lib.genbmm_logbmm_bwdbwd_ws(P(wide[0]), P(wide[1]), P(wide[2]), P(wide[3]), P(w_a), P(w_b), P(ga32),
                                           P(gb32), P(gg32), P(ws32), B, M, K, N, s) == 0
        assert torch.equal(ga, ga32.to(dt)) and torch.equal(gb, gb32.to(dt)) and torch.equal(gg, gg32.to(dt))
    # the workspace is required for the half types
    assert getattr(lib, "genbmm_logbmm_bwdbwd_ws" + suffix)(P(a), P(b), P(out), P(g), P(ua), P(ub), P(ga), P(gb), P(gg),
                                                           P(None), B, M, K, N, s) == -1
