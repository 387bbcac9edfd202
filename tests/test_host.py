"""Host-side logic that needs no GPU: band structure operations against explicit index
loops (the reference's test_sparse.py strategy), the C-ABI library's exported symbols,
and the no-CPU-fallback rule."""
import ctypes
import os
import re

import pytest
import torch
from hypothesis import given, settings
from hypothesis.strategies import integers

import oracle
import genbmm_amd
from genbmm_amd import _lib
from genbmm_amd.sparse import BandedMatrix, banddiag

mint = integers(min_value=6, max_value=10)
lint = integers(min_value=0, max_value=10)
sint = integers(min_value=3, max_value=5)
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@settings(max_examples=25, deadline=None)
@given(sint, mint, lint, lint)
def test_band_structure(batch, n, lu, ld):
    """Mirrors genbmm/test_sparse.py:12-55 with the loops living in the oracle."""
    start = torch.rand(batch, n, n)
    band, same = banddiag(start, lu, ld)
    assert torch.equal(band, oracle.band_from_dense(start, lu, ld))
    assert torch.equal(same, start)
    mid = oracle.band_to_dense(band, lu, ld, 0.0)
    banded = BandedMatrix(band, lu, ld)
    assert torch.equal(banded.to_dense(), mid)
    assert torch.equal(BandedMatrix(band, lu, ld, fill=-3.0).to_dense(), oracle.band_to_dense(band, lu, ld, -3.0))
    t = banded.transpose()
    assert (t.lu, t.ld) == (ld, lu)
    assert torch.equal(t.to_dense(), mid.transpose(-2, -1))
    assert torch.equal(t.data, oracle.band_transpose(band, lu, ld))
    plus = banded.op(banded, lambda a, b: a + b)
    assert (plus.lu, plus.ld) == (lu, ld)
    assert torch.equal(plus.data, band + band) and torch.equal(plus.to_dense(), mid + mid)
    plus = banded.op(banded.transpose(), lambda a, b: a + b)
    assert plus.lu == max(lu, ld) and plus.ld == max(lu, ld)
    assert torch.equal(plus.to_dense(), mid.transpose(-2, -1) + mid)
    wide = banded._expand(lu + 2, ld + 1)
    assert torch.equal(wide.to_dense(), mid)


@settings(max_examples=15, deadline=None)
@given(sint, mint)
def test_col_shift(batch, n):
    """genbmm/test_sparse.py:87-107."""
    lu = ld = 1
    band, _ = banddiag(torch.rand(batch, n, n), lu, ld)
    bx = BandedMatrix(band, lu, ld)
    x = bx.to_dense()
    x2 = torch.cat([x[:, :, 1:], torch.zeros(batch, n, 1)], 2)
    assert torch.equal(banddiag(x2, lu - 1, ld + 1)[0], bx.col_shift(1).data)
    x2 = torch.cat([torch.zeros(batch, n, 1), x[:, :, :-1]], 2)
    assert torch.equal(banddiag(x2, lu + 1, ld - 1)[0], bx.col_shift(-1).data)
    assert torch.equal(bx.col_unshift().data, bx.col_shift(-1).data)
    assert bx.col_shift(0) is bx and bx.band_shift(0) is bx and bx.band_pad(0) is bx


def test_band_relabel_ops():
    """band_shift / band_pad / band_unshift are pure relabelling of the same cells
    (sparse.py:96-152): checked here on the dense matrix they denote, and further down
    against the reference's own outputs."""
    band, _ = banddiag(torch.rand(2, 7, 7), 2, 3)
    bx = BandedMatrix(band, 2, 3, fill=0)
    x = bx.to_dense()
    p = bx.band_pad(2)
    assert (p.lu, p.ld, p.width) == (4, 5, 10) and torch.equal(p.to_dense(), x)
    s = bx.band_shift(1)     # drops band cell 0, relabels lu+1 / ld-1
    assert (s.lu, s.ld) == (3, 2)
    assert torch.equal(s.data[:, :, :-1], band[:, :, 1:]) and bool((s.data[:, :, -1] == 0).all())
    s = bx.band_shift(-2)
    assert (s.lu, s.ld) == (0, 5)
    assert torch.equal(s.data[:, :, 2:], band[:, :, :-2]) and bool((s.data[:, :, :2] == 0).all())
    u = bx.band_unshift()
    assert (u.lu, u.ld) == (1, 4) and torch.equal(u.data, bx.band_shift(-1).data)
    f = BandedMatrix(band, 2, 3, fill=-1e9).band_pad(1)
    assert bool((f.data[:, :, 0] == -1e9).all()) and bool((f.data[:, :, -1] == -1e9).all())


def test_transpose_is_differentiable():
    band = banddiag(torch.rand(2, 6, 6), 2, 1)[0].clone().requires_grad_(True)
    t = BandedMatrix(band, 2, 1).transpose()
    (g,) = torch.autograd.grad(t.data.sum(), band)
    inside = oracle.band_from_dense(torch.ones(2, 6, 6), 2, 1)
    assert torch.equal(g, inside)


def test_module_level_names_of_the_reference():
    """has_cuda, repdiag, Transpose / Transpose2 (sparse.py:3-9, 33-77): repdiag against its
    definition by padding and diagonals, Transpose against the dense transpose."""
    from genbmm_amd import sparse

    assert sparse.has_cuda == os.path.exists(_lib.LIB_PATH)
    torch.manual_seed(4)
    x, lu, ld = torch.randn(2, 7, 6), 2, 3
    want = torch.zeros(2, 7, 6)
    for i in range(7):
        for j in range(6):
            if 0 <= i + j - ld < 7:
                want[:, i, j] = x[:, i + j - ld, j]
    assert torch.equal(sparse.repdiag(x, lu, ld), want)
    dense = torch.randn(2, 7, 7)
    band = banddiag(dense, lu, ld)[0].clone().requires_grad_(True)
    t = sparse.Transpose.apply(band, lu, ld)
    assert torch.equal(t, banddiag(dense.transpose(1, 2), ld, lu)[0])
    (g,) = torch.autograd.grad((t * t).sum(), band, create_graph=True)
    inside = oracle.band_from_dense(torch.ones(2, 7, 7), lu, ld)
    assert torch.allclose(g, 2 * band * inside)
    (gg,) = torch.autograd.grad(g.sum(), band)
    assert torch.allclose(gg, 2 * inside)
    assert sparse.Transpose2 is sparse.Transpose


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "genbmm_gfx950.h")).read()
    declared = set(re.findall(r"\b(genbmm_[a-z_0-9]+)\s*\(", header))
    assert len(declared) == 76
    assert declared == set(_lib.SIGNATURES) | set(_lib.STRING_FUNCS) | set(_lib.SIZE_FUNCS) | set(_lib.INT_FUNCS)
    assert os.path.exists(_lib.LIB_PATH), "build with `python -m genbmm_amd.build`"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    lib.genbmm_version.restype = ctypes.c_char_p
    assert lib.genbmm_version().startswith(b"genbmm-gfx950")
    lib.genbmm_error_string.restype = ctypes.c_char_p
    assert lib.genbmm_error_string(-2) == b"a dimension is negative or too large"


def test_banded_workspace_and_scratch_sizes_agree_on_the_backward_path():
    """The log product's workspace holds a place for H = g / S exactly when the backward is not
    the memory-fed one (which forms H on the fly and needs no scratch either): for every band
    shape, either workspace = rows * (Wa + Wb + Wo + 2) and scratch = 0, or the workspace has
    Wo more floats per row and scratch is 0 (workspace unused) or rows * Wo.  Host code only."""
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in ("genbmm_banded_workspace_size", "genbmm_banded_scratch_size"):
        getattr(lib, name).restype = ctypes.c_size_t
        getattr(lib, name).argtypes = [ctypes.c_int] * 6
    B, n = 3, 500
    rows = B * n
    lean = full = 0
    widths = list(range(0, 9)) + [15, 16, 32, 48, 60, 100, 110, 111, 112, 113, 120, 127, 128, 140]
    for lu in widths:
        for ld in (lu, max(lu - 1, 0), 0):
            for blu, bld in ((lu, ld), (1, 2), (ld, lu)):
                Wa, Wb = lu + ld + 1, blu + bld + 1
                Wo = Wa + Wb - 1
                ws = lib.genbmm_banded_workspace_size(lu, ld, blu, bld, B, n)
                sc = lib.genbmm_banded_scratch_size(lu, ld, blu, bld, B, n)
                if ws == rows * (Wa + Wb + Wo + 2):
                    assert sc == 0, (lu, ld, blu, bld)
                    lean += 1
                else:
                    assert ws == rows * (Wa + Wb + 2 * Wo + 2), (lu, ld, blu, bld)
                    assert sc in (0, rows * Wo), (lu, ld, blu, bld)
                    full += 1
    assert lean > 20 and full > 5
    assert lib.genbmm_banded_workspace_size(-1, 0, 0, 0, B, n) == 0


def test_launch_grids_beyond_32_bits_are_refused():
    """Shapes whose launch grid would exceed 2^31 - 1 workgroups (and wrap silently) return
    GENBMM_E_SHAPE before anything is launched or any pointer is read.  Host code only."""
    lib = _lib.load()
    fake = ctypes.c_void_p(256)      # never dereferenced: the shape check comes first
    E_SHAPE = -2
    # banded: 2^30 batch items of 64 rows -> 2^32 tile rows
    for mode in (0, 1, 3):
        assert lib.genbmm_banded_fwd(fake, 1, 1, fake, 1, 1, fake, fake, None, 1 << 30, 64, mode, None) == E_SHAPE
    assert lib.genbmm_banded_bwd(fake, 1, 1, fake, 1, 1, fake, fake, None, fake, fake, fake, 1 << 30, 64, 3, None) == E_SHAPE
    assert lib.genbmm_banded_sample_fwd(fake, 1, 1, fake, 1, 1, fake, fake, None, 1, 0, 1 << 30, 64, None) == E_SHAPE
    # dense: 2^37 result cells pass the element count, their 2^32 tiles of 32 x 32 do not
    B, M, K, N = 1 << 20, 1, 1, 1 << 17
    assert lib.genbmm_maxbmm_fwd(fake, fake, fake, fake, B, M, K, N, None) == E_SHAPE
    assert lib.genbmm_logbmm_fwd(fake, fake, fake, None, B, M, K, N, None) == E_SHAPE
    assert lib.genbmm_logbmm_bwd(fake, fake, fake, fake, None, fake, fake, B, M, K, N, None) == E_SHAPE
    assert lib.genbmm_samplebmm_fwd(fake, fake, fake, fake, None, 1, 0, B, M, K, N, None) == E_SHAPE
    assert lib.genbmm_argmax_bwd(fake, fake, fake, fake, B, M, K, N, None) == E_SHAPE
    assert lib.genbmm_logbmm_fwd_f64(fake, fake, fake, B, M, K, N, None) == E_SHAPE
    # an ordinary large problem is still accepted by the size functions
    assert lib.genbmm_logbmm_stats_size(64, 512, 512, 512) > 0


def test_half_builds_compute_in_float():
    """The float16 / bfloat16 builds of the dense sources widen on load and narrow on store
    and do nothing else in the narrow type: their device code (LLVM IR) holds no arithmetic,
    comparison or min / max on half or bfloat values, scalar or vector."""
    import shutil
    import subprocess
    from concurrent.futures import ThreadPoolExecutor
    from genbmm_amd import build as hip_build
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not present")
    jobs = [(src, elem) for src, variants in hip_build.PER_ELEMENT.items() for _, elem in variants if elem]
    assert len(jobs) == 10

    def ir(job):
        src, elem = job
        cmd = [hipcc, "-O1", "-std=c++17", "--offload-arch=gfx950", "-ffp-contract=on", "-fno-gpu-rdc",
               "-DGENBMM_ELEM=%d" % elem, "-S", "-emit-llvm", "--cuda-device-only", "-o", "-",
               os.path.join(hip_build.CSRC, src)]
        return subprocess.run(cmd, check=True, capture_output=True, text=True).stdout

    narrow = re.compile(r"= (fadd|fsub|fmul|fdiv|frem|fneg|fcmp \w+) [^\n]*?(<\d+ x )?(half|bfloat)\b"
                        r"|call [^\n]*llvm\.(maxnum|minnum|fma|fmuladd|maximum|minimum)\.(v\d+)?(f16|bf16)")
    with ThreadPoolExecutor(max_workers=8) as pool:
        for job, text in zip(jobs, pool.map(ir, jobs)):
            assert "define" in text and ("half" in text or "bfloat" in text), job
            hits = [m.group(0) for m in narrow.finditer(text)]
            assert not hits, (job, hits[:3])


def test_no_cpu_fallback():
    a, b = torch.randn(2, 3, 4), torch.randn(2, 4, 5)
    for op in (genbmm_amd.logbmm, genbmm_amd.maxbmm, genbmm_amd.samplebmm, genbmm_amd.prodmaxbmm):
        with pytest.raises(RuntimeError):
            op(a, b)
    band = torch.randn(2, 5, 3)
    for name in ("multiply", "multiply_log", "multiply_max"):
        with pytest.raises(RuntimeError):
            getattr(BandedMatrix(band, 1, 1), name)(BandedMatrix(band, 1, 1))


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "genbmm_amd")
    for fn in os.listdir(pkg):
        if fn.endswith(".py"):
            src = open(os.path.join(pkg, fn)).read()
            assert not re.search(r"^\s*(import|from)\s+oracle\b", src, re.M), fn


def test_install_as_genbmm():
    import sys

    mod = genbmm_amd.install_as_genbmm()
    import genbmm

    assert genbmm is mod and genbmm.logbmm is genbmm_amd.logbmm
    from genbmm.sparse import BandedMatrix as BM

    assert BM is BandedMatrix
    for k in ("genbmm", "genbmm.genmul", "genbmm.sparse"):
        sys.modules.pop(k, None)


# ---------------------------------------------------------------- golden fixtures
# tests/golden/band_struct.npz holds input / output vectors written by running the
# reference's own pure-Python BandedMatrix methods (sparse.py:81-218) on the CPU
# (tests/golden/make_band_struct_fixtures.py): the reference has no test for them.
GOLDEN = os.path.join(ROOT, "tests", "golden", "band_struct.npz")


def _golden():
    import numpy as np

    return np.load(GOLDEN, allow_pickle=False)


@pytest.mark.parametrize("case", range(4))
def test_band_structural_ops_match_reference_vectors(case):
    z = _golden()
    p = "c%d_" % case
    B, n, lu, ld, olu, old = (int(v) for v in z[p + "meta"])
    fill = float(z[p + "fill"])
    bm = BandedMatrix(torch.from_numpy(z[p + "band"]), lu, ld, fill)
    om = BandedMatrix(torch.from_numpy(z[p + "oband"]), olu, old, fill)

    def same(name, m):
        assert [m.lu, m.ld] == [int(v) for v in z[p + name + "_luld"]], name
        assert torch.equal(m.data, torch.from_numpy(z[p + name])), name

    same("band_shift_p1", bm.band_shift(1))
    same("band_shift_m2", bm.band_shift(-2))
    same("band_pad_2", bm.band_pad(2))
    same("band_unshift", bm.band_unshift())
    same("col_shift_p1", bm.col_shift(1))
    same("col_shift_m2", bm.col_shift(-2))
    same("col_unshift", bm.col_unshift())
    same("expand", bm._expand(lu + 2, ld + 1))
    same("op_add", bm.op(om, lambda x, y: x + y, zero=0))
    same("op_max", bm.op(om, torch.max, zero=-1e9))
    same("transpose", bm.transpose())
    assert torch.equal(bm.to_dense(), torch.from_numpy(z[p + "to_dense"]))


def test_three_bf16_parts_of_a_float_add_up_to_it_exactly():
    """The arithmetic behind the default logbmm kernels' products (genbmm_amd/csrc/logbmm_split.h):
    a float x is cut into three bfloat16 parts by rounding and subtracting twice; the parts add up
    to x exactly (8 + 8 + 8 significant bits; below 2^-100 the last part can fall into the
    denormals, far beneath any factor the kernels' guard lets matter), and the six partial
    products the kernels take - all but m l, l m, l l - give x y within 2^-22 of it: the size of
    the rounding of one fp32 product."""
    import torch
    torch.manual_seed(0)
    mag = torch.exp2(torch.empty(400000).uniform_(-60.0, 60.0))
    x = torch.cat([torch.rand(200000), torch.randn(200000) * 1e3, mag * torch.sign(torch.randn(400000)),
                   torch.tensor([0.0, 1.0, 2.0 ** -40, 1 - 2.0 ** -24, 3.0e38, -7.25])])

    def parts(v):
        h = v.bfloat16().float()
        r = v - h
        m = r.bfloat16().float()
        l = (r - m).bfloat16().float()
        return h, m, l

    h, m, l = parts(x)
    assert torch.equal((h.double() + m.double()) + l.double(), x.double())
    y = x[torch.randperm(x.numel())]
    hy, my, ly = parts(y)
    d = lambda t: t.double()
    six = d(h) * d(hy) + d(h) * d(my) + d(m) * d(hy) + d(m) * d(my) + d(h) * d(ly) + d(l) * d(hy)
    exact = d(x) * d(y)
    fin = torch.isfinite(exact) & (exact != 0)
    rel = ((six - exact).abs() / exact.abs())[fin]
    assert float(rel.max()) <= 2.0 ** -22, float(rel.max())
