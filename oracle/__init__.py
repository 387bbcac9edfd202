"""TEST INFRASTRUCTURE ONLY - CPU oracle for the genbmm hot path.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; genbmm_amd/ never does.

Two layers:

* closed forms in PyTorch on the CPU - the reference's own CPU formulation, the
  broadcast identities of README.md:23-66 and genbmm/test_cuda.py:17, and the
  dense identities of genbmm/test_sparse.py for banded matrices;
* `seq_*` - ctypes wrappers of oracle/seq_oracle.c, a sequential plain-C
  restatement of every reference kernel (float and double instantiations) and
  of Philox4x32-10.

What pins the oracle itself is listed in tests/test_oracle.py.  The reference
has no stored vectors for this path and cannot be built here (CUDA only), so
there is no oracle/_ref; the band products are additionally pinned by vectors
that the reference's own CPU loops produced (tests/golden/band_struct.npz).
Parity unpinned: only the random stream of samplebmm (the reference draws from
torch's CUDA generator); its decision rule and distribution are pinned.  The
banded sample product has no reference function at all (the reference's band
kernel has no sample mode): its restatement is the reference's dense sampling
rule on a band cell's terms and is pinned through the dense sampling oracle on
the equivalent dense operands, not against the reference.
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "liboracle.so")
_lib = None


def build():
    """Compile oracle/seq_oracle.c with gcc (always rebuilds)."""
    subprocess.run(["make", "-s", "-B", "-C", _HERE], check=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _np(t, dtype):
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().numpy()
    return np.ascontiguousarray(t, dtype=dtype)


def _p(x):
    return x.ctypes.data_as(ctypes.c_void_p) if x is not None else ctypes.c_void_p(0)


def _prefix(dtype):
    return ("orc_d_", np.float64) if dtype in (np.float64, torch.float64, "d") else ("orc_f_", np.float32)


# ===================================================================== closed forms
def logbmm_broadcast(a, b):
    """README.md:31-35 / test_cuda.py:17."""
    return (a.unsqueeze(-1) + b.unsqueeze(-3)).logsumexp(-2)


def maxbmm_broadcast(a, b):
    """README.md:41-44; returns (values, indices); torch's CPU max keeps the first maximum."""
    r = (a.unsqueeze(-1) + b.unsqueeze(-3)).max(-2)
    return r.values, r.indices


def prodmaxbmm_broadcast(a, b):
    """README.md:60-63."""
    r = (a.unsqueeze(-1) * b.unsqueeze(-3)).max(-2)
    return r.values, r.indices


def logbmm_grads64(a, b, g):
    """float64 autograd through the broadcast form (test_cuda.py:22-27)."""
    a = a.detach().double().requires_grad_(True)
    b = b.detach().double().requires_grad_(True)
    out = logbmm_broadcast(a, b)
    ga, gb = torch.autograd.grad(out, (a, b), g.double())
    return out.detach(), ga, gb


def logbmm_second_order64(a, b, g, u_a, u_b):
    """Gradients of <u_a, grad_a> + <u_b, grad_b> w.r.t. (a, b, g), float64 autograd
    with create_graph (test_cuda.py:30-39)."""
    a = a.detach().double().requires_grad_(True)
    b = b.detach().double().requires_grad_(True)
    g = g.detach().double().requires_grad_(True)
    out = logbmm_broadcast(a, b)
    ga, gb = torch.autograd.grad(out, (a, b), g, create_graph=True)
    outs, cots = [], []
    if u_a is not None:
        outs.append(ga)
        cots.append(u_a.double())
    if u_b is not None:
        outs.append(gb)
        cots.append(u_b.double())
    return torch.autograd.grad(outs, (a, b, g), cots)


def sample_cdf64(a, b):
    """Inclusive CDF over k of softmax_k(a[m,k] + b[k,n]) in float64, shape (B,M,K,N)."""
    s = a.double().unsqueeze(-1) + b.double().unsqueeze(-3)
    return torch.softmax(s, dim=-2).cumsum(-2)


def sample_index_from_cdf(cdf, u):
    """Reference rule (matmul_cuda_kernel.cu:109-118): first k with C[k-1] < r and
    C[k] > r; 0 if there is none.  cdf (B,M,K,N) inclusive, u (B,M,N)."""
    r = u.double().unsqueeze(-2)
    prev = torch.cat([torch.zeros_like(cdf[..., :1, :]), cdf[..., :-1, :]], dim=-2)
    hit = (prev < r) & (cdf > r)
    first = hit.to(torch.int8).argmax(-2)
    return torch.where(hit.any(-2), first, torch.zeros_like(first)).to(torch.int32)


# ===================================================================== Philox
def philox4x32_10(ctr, key):
    c = (ctypes.c_uint32 * 4)(*ctr)
    k = (ctypes.c_uint32 * 2)(*key)
    o = (ctypes.c_uint32 * 4)()
    lib().orc_philox4x32_10(c, k, o)
    return tuple(int(x) for x in o)


def philox4x32_10_py(ctr, key):
    """Independent pure-Python-int implementation of the published algorithm."""
    c0, c1, c2, c3 = ctr
    k0, k1 = key
    mask = 0xFFFFFFFF
    for _ in range(10):
        p0 = 0xD2511F53 * c0
        p1 = 0xCD9E8D57 * c2
        c0, c1, c2, c3 = ((p1 >> 32) ^ c1 ^ k0) & mask, p1 & mask, ((p0 >> 32) ^ c3 ^ k1) & mask, p0 & mask
        k0 = (k0 + 0x9E3779B9) & mask
        k1 = (k1 + 0xBB67AE85) & mask
    return c0, c1, c2, c3


def philox_uniform(first, count, seed, offset):
    out = np.empty(count, dtype=np.float32)
    fn = lib().orc_philox_uniform
    fn.argtypes = [ctypes.c_uint64] * 4 + [ctypes.c_void_p]
    fn(first, count, seed, offset, _p(out))
    return torch.from_numpy(out)


# ===================================================================== sequential C
def _dims(a, b):
    B, M, K = a.shape
    return B, M, K, b.shape[2]


def seq_logbmm_fwd(a, b, dtype=np.float32):
    pre, dt = _prefix(dtype)
    a, b = _np(a, dt), _np(b, dt)
    B, M, K, N = _dims(a, b)
    out, mx = np.empty((B, M, N), dt), np.empty((B, M, N), dt)
    getattr(lib(), pre + "logbmm_fwd")(_p(a), _p(b), _p(out), _p(mx), B, M, K, N)
    return torch.from_numpy(out), torch.from_numpy(mx)


def seq_maxbmm_fwd(a, b, prod=False, dtype=np.float32):
    pre, dt = _prefix(dtype)
    a, b = _np(a, dt), _np(b, dt)
    B, M, K, N = _dims(a, b)
    out, idx = np.empty((B, M, N), dt), np.empty((B, M, N), np.int32)
    getattr(lib(), pre + "maxbmm_fwd")(_p(a), _p(b), _p(out), _p(idx), B, M, K, N, int(prod))
    return torch.from_numpy(out), torch.from_numpy(idx)


def seq_samplebmm_fwd(a, b, rnd, dtype=np.float32):
    pre, dt = _prefix(dtype)
    a, b, rnd = _np(a, dt), _np(b, dt), _np(rnd, dt)
    B, M, K, N = _dims(a, b)
    out, idx = np.empty((B, M, N), dt), np.empty((B, M, N), np.int32)
    getattr(lib(), pre + "samplebmm_fwd")(_p(a), _p(b), _p(rnd), _p(out), _p(idx), B, M, K, N)
    return torch.from_numpy(out), torch.from_numpy(idx)


def seq_logbmm_bwd(a, b, g, dtype=np.float32):
    pre, dt = _prefix(dtype)
    a, b, g = _np(a, dt), _np(b, dt), _np(g, dt)
    B, M, K, N = _dims(a, b)
    out, mx = np.empty((B, M, N), dt), np.empty((B, M, N), dt)
    getattr(lib(), pre + "logbmm_fwd")(_p(a), _p(b), _p(out), _p(mx), B, M, K, N)
    ga, gb = np.empty_like(a), np.empty_like(b)
    getattr(lib(), pre + "logbmm_bwd")(_p(a), _p(b), _p(out), _p(mx), _p(g), _p(ga), _p(gb), B, M, K, N)
    return torch.from_numpy(ga), torch.from_numpy(gb)


def seq_logbmm_bwdbwd(a, b, g, u, dtype=np.float32):
    """The reference's literal quartic kernels: grads of <u, grad_a> w.r.t. (a, b, g)."""
    pre, dt = _prefix(dtype)
    a, b, g, u = _np(a, dt), _np(b, dt), _np(g, dt), _np(u, dt)
    B, M, K, N = _dims(a, b)
    out, mx = np.empty((B, M, N), dt), np.empty((B, M, N), dt)
    getattr(lib(), pre + "logbmm_fwd")(_p(a), _p(b), _p(out), _p(mx), B, M, K, N)
    ga, gb, gg = np.empty_like(a), np.empty_like(b), np.empty_like(g)
    getattr(lib(), pre + "logbmm_bwdbwd")(_p(a), _p(b), _p(out), _p(mx), _p(g), _p(u),
                                          _p(ga), _p(gb), _p(gg), B, M, K, N)
    return torch.from_numpy(ga), torch.from_numpy(gb), torch.from_numpy(gg)


def seq_argmax_bwd(a, b, idx, g, prod=False, dtype=np.float32):
    pre, dt = _prefix(dtype)
    g, idx = _np(g, dt), _np(idx, np.int32)
    B, M, N = g.shape
    if prod:
        a, b = _np(a, dt), _np(b, dt)
        K = a.shape[2]
    else:
        K = a if isinstance(a, int) else a.shape[2]
        a = b = None
    ga, gb = np.empty((B, M, K), dt), np.empty((B, K, N), dt)
    getattr(lib(), pre + "argmax_bwd")(_p(a), _p(b), _p(idx), _p(g), _p(ga), _p(gb), B, M, K, N, int(prod))
    return torch.from_numpy(ga), torch.from_numpy(gb)


# ===================================================================== banded
def band_from_dense(x, lu, ld):
    """Explicit loops of genbmm/test_sparse.py:18-24: band[:, c, lu - c + r] = x[:, r, c]."""
    x = x.detach().cpu()
    batch, n, _ = x.shape
    band = torch.zeros(batch, n, lu + ld + 1, dtype=x.dtype)
    for r in range(n):
        for c in range(n):
            if c == r or (r < c and c - r <= lu) or (r > c and r - c <= ld):
                band[:, c, lu - c + r] = x[:, r, c]
    return band


def band_to_dense(data, lu, ld, fill=0.0):
    """Inverse of band_from_dense; cells outside the band hold `fill` (test_sparse.py:27-35)."""
    data = data.detach().cpu()
    batch, n, _ = data.shape
    full = torch.full((batch, n, n), float(fill), dtype=data.dtype)
    for r in range(n):
        for c in range(n):
            if c == r or (r < c and c - r <= lu) or (r > c and r - c <= ld):
                full[:, r, c] = data[:, c, lu - c + r]
    return full


def band_transpose(data, lu, ld):
    """Band data (lu' = ld, ld' = lu) of the transposed matrix, through the dense form."""
    return band_from_dense(band_to_dense(data, lu, ld, 0.0).transpose(-2, -1), ld, lu)


def band_transpose_indexed(data, lu, ld):
    """The same transposition by index arithmetic, for sizes where the dense detour is
    too slow: T[i, k] = data[i + k - ld, W - 1 - k] where that row exists, else 0
    (from the layout: T[c, k] = Dense[c, c + k - ld]).  Pinned against band_transpose
    in tests/test_oracle.py."""
    d = _np(data, np.float64 if data.dtype == torch.float64 else np.float32)
    n, W = d.shape[1], d.shape[2]
    i = np.arange(n)[:, None]
    k = np.arange(W)[None, :]
    src = i + k - ld
    ok = (src >= 0) & (src < n)
    out = d[:, np.clip(src, 0, n - 1), np.broadcast_to(W - 1 - k, src.shape)]
    return torch.from_numpy(np.where(ok[None], out, 0).astype(d.dtype))


def band_relabel(data, dcol, dband, w_out, fill):
    """out[b, c, k] = data[b, c + dcol, k + dband] where that cell exists, else `fill`:
    the one index rule behind the reference's slicing-and-padding methods
    (genbmm/sparse.py): band_shift(t) :96-110 is dband = t; band_pad(t) :112-123 is
    dband = -|t| with 2|t| more cells; band_unshift :137-152 is dband = -1;
    col_shift(t) :154-165 is dcol = t; col_unshift :167-182 is dcol = -1; _expand
    :192-197 is dband = -(lu' - lu).  Explicit loops; pinned against the reference's own
    outputs (tests/golden/band_struct.npz) in tests/test_oracle.py."""
    d = data.detach().cpu().numpy()
    batch, n, w = d.shape
    out = np.full((batch, n, w_out), fill, dtype=d.dtype)
    for c in range(n):
        cs = c + dcol
        if cs < 0 or cs >= n:
            continue
        for k in range(w_out):
            ks = k + dband
            if 0 <= ks < w:
                out[:, c, k] = d[:, cs, ks]
    return torch.from_numpy(out)


def band_op(a, a_lu, a_ld, b, b_lu, b_ld, fn, zero):
    """BandedMatrix.op (genbmm/sparse.py:199-212) cell by cell on the union band:
    `zero` where neither operand has a cell, a's value where only a has one,
    fn(zero, b) where only b has one, fn(a, b) where both do.  `fn` works on numpy
    arrays.  Returns (data, lu, ld)."""
    x, y = a.detach().cpu().numpy(), b.detach().cpu().numpy()
    batch, n, wa = x.shape
    wb = y.shape[2]
    lu, ld = max(a_lu, b_lu), max(a_ld, b_ld)
    out = np.full((batch, n, lu + ld + 1), zero, dtype=x.dtype)
    for k in range(lu + ld + 1):
        ka, kb = k - (lu - a_lu), k - (lu - b_lu)
        cur = x[:, :, ka] if 0 <= ka < wa else out[:, :, k]
        out[:, :, k] = fn(cur, y[:, :, kb]) if 0 <= kb < wb else cur
    return torch.from_numpy(out), lu, ld


def band_product_dense(a, a_lu, a_ld, b, b_lu, b_ld, mode):
    """X.multiply*(Y) as dense algebra (test_sparse.py:141-142, 181-195): Dense(Y)^T (x)
    Dense(X), re-banded with lu = a_lu + b_ld, ld = a_ld + b_lu.  mode 3: torch.bmm;
    mode 0 / 1: logsumexp / max over p of Y[p,r] + X[p,c] with -1e9 outside the bands.
    Returns (band, in_matrix_mask)."""
    fill = 0.0 if mode == 3 else -1e9
    X = band_to_dense(a, a_lu, a_ld, fill)
    Y = band_to_dense(b, b_lu, b_ld, fill)
    if mode == 3:
        D = torch.bmm(Y.transpose(-2, -1), X)
    else:
        S = Y.transpose(-2, -1).unsqueeze(-1) + X.unsqueeze(-3)  # [r, p, c]
        D = S.logsumexp(-2) if mode == 0 else S.max(-2).values
    lu, ld = a_lu + b_ld, a_ld + b_lu
    n = a.shape[1]
    mask = band_from_dense(torch.ones(1, n, n), lu, ld)[0] > 0
    return band_from_dense(D, lu, ld), mask


def seq_band_fwd(a, a_lu, a_ld, b, b_lu, b_ld, mode, dtype=np.float32):
    pre, dt = _prefix(dtype)
    a, b = _np(a, dt), _np(b, dt)
    B, n, _ = a.shape
    W = a.shape[2] + b.shape[2] - 1
    out, idx, mx = np.empty((B, n, W), dt), np.empty((B, n, W), np.int32), np.empty((B, n, W), dt)
    getattr(lib(), pre + "band_fwd")(_p(a), a_lu, a_ld, _p(b), b_lu, b_ld, _p(out), _p(idx), _p(mx), B, n, mode)
    return torch.from_numpy(out), torch.from_numpy(idx), torch.from_numpy(mx)


def seq_band_sample_fwd(a, a_lu, a_ld, b, b_lu, b_ld, rnd, dtype=np.float32):
    """Banded sample product: (out, idx) for the uniforms `rnd` (B, n, Wo)."""
    pre, dt = _prefix(dtype)
    a, b, rnd = _np(a, dt), _np(b, dt), _np(rnd, dt)
    B, n, _ = a.shape
    W = a.shape[2] + b.shape[2] - 1
    out, idx = np.empty((B, n, W), dt), np.empty((B, n, W), np.int32)
    getattr(lib(), pre + "band_sample_fwd")(_p(a), a_lu, a_ld, _p(b), b_lu, b_ld, _p(rnd), _p(out), _p(idx), B, n)
    return torch.from_numpy(out), torch.from_numpy(idx)


def band_pairs(a, a_lu, a_ld, b, b_lu, b_ld):
    """The factor pairs of every band cell, by index arithmetic (works on any device, keeps
    the dtype, differentiable): av[b, i, j, k] = a[b, i, k], bv[b, i, j, k] = b[b, o, k2] with
    o = i + j - lu_out, k2 = k - j + Wb - 1, and valid[i, j, k] = 0 <= o < n and 0 <= k2 < Wb
    and 0 <= i + k - a_lu < n (banded_cuda_kernel.cu:32-51).  bv holds an arbitrary cell of b
    where not valid."""
    B, n, Wa = a.shape
    Wb = b.shape[2]
    Wo, r_lu = Wa + Wb - 1, a_lu + b_ld
    dev = a.device
    i = torch.arange(n, device=dev).view(n, 1, 1)
    j = torch.arange(Wo, device=dev).view(1, Wo, 1)
    k = torch.arange(Wa, device=dev).view(1, 1, Wa)
    o, k2, pos = i + j - r_lu, k - j + (Wb - 1), i + k - a_lu
    valid = (o >= 0) & (o < n) & (k2 >= 0) & (k2 < Wb) & (pos >= 0) & (pos < n)
    bv = b[:, o.clamp(0, n - 1).expand(n, Wo, Wa), k2.clamp(0, Wb - 1).expand(n, Wo, Wa)]
    return a.unsqueeze(2).expand(B, n, Wo, Wa), bv, valid


def band_terms64(a, a_lu, a_ld, b, b_lu, b_ld):
    """Every term a[i, k] + b[o, k2] of every band cell in float64, (B, n, Wo, Wa), -inf where
    the pair is not valid.  Returns (v, valid)."""
    av, bv, valid = band_pairs(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld)
    v = av + bv
    return torch.where(valid, v, torch.full_like(v, -float("inf"))), valid


def band_product64(a, a_lu, a_ld, b, b_lu, b_ld, mode):
    """The banded product as a closed form over band_pairs in float64 (any device,
    differentiable in a and b): mode 3 sum of products, mode 0 log-sum-exp of sums; cells
    outside the matrix are 0.  The same arithmetic as band_product_dense without the dense
    detour, for sizes where that is too large; pinned against it in tests/test_oracle.py."""
    av, bv, valid = band_pairs(a.double(), a_lu, a_ld, b.double(), b_lu, b_ld)
    inside = valid.any(-1)
    if mode == 3:
        return torch.where(valid, av * bv, torch.zeros_like(av)).sum(-1)
    v = torch.where(valid, av + bv, torch.full_like(av, -float("inf")))
    v = torch.where(inside.unsqueeze(-1), v, torch.zeros_like(v))
    return torch.where(inside, v.logsumexp(-1), torch.zeros_like(v[..., 0]))


def band_max_first(a, a_lu, a_ld, b, b_lu, b_ld):
    """Max-plus band product in the operands' own dtype (one rounding per sum, as the
    reference) with the lowest k that attains the maximum, any device: (values, idx);
    cells outside the matrix are 0 / 0.  Assumes every cell has a term above the -1e9
    floor (banded_cuda_kernel.cu:79)."""
    av, bv, valid = band_pairs(a, a_lu, a_ld, b, b_lu, b_ld)
    inside = valid.any(-1)
    v = torch.where(valid, av + bv, torch.full_like(av, -float("inf")))
    m = v.max(-1).values
    k = torch.arange(a.shape[2], device=a.device).expand_as(v)
    first = torch.where(v == m.unsqueeze(-1), k, torch.full_like(k, a.shape[2])).min(-1).values
    return torch.where(inside, m, torch.zeros_like(m)), torch.where(inside, first, torch.zeros_like(first)).to(torch.int32)


def band_sample_cdf64(a, a_lu, a_ld, b, b_lu, b_ld):
    """Inclusive CDF over k of softmax_k of a band cell's terms, float64, (B, n, Wo, Wa);
    cells outside the matrix (no term) hold zeros."""
    v, valid = band_terms64(a, a_lu, a_ld, b, b_lu, b_ld)
    has = valid.any(-1, keepdim=True)
    p = torch.softmax(torch.where(has, v, torch.zeros_like(v)), -1)
    return torch.where(has & valid, p, torch.zeros_like(p)).cumsum(-1), valid


def band_sample_index_from_cdf(cdf, valid, u):
    """The dense rule (matmul_cuda_kernel.cu:109-118) on a band cell's CDF: first k with
    C[k-1] < r and C[k] > r; the cell's first term if there is none; 0 outside the matrix."""
    r = u.double().unsqueeze(-1)
    prev = torch.cat([torch.zeros_like(cdf[..., :1]), cdf[..., :-1]], dim=-1)
    hit = valid & (prev < r) & (cdf > r)
    first_hit = hit.to(torch.int8).argmax(-1)
    first_term = valid.to(torch.int8).argmax(-1).expand_as(first_hit)
    return torch.where(hit.any(-1), first_hit, first_term).to(torch.int32)


def _seq_band_bwd_first(pre, dt, a, a_lu, a_ld, b, b_lu, b_ld, part, g, mode):
    a, b, part, g = _np(a, dt), _np(b, dt), _np(part, dt), _np(g, dt)
    B, n, _ = a.shape
    ga = np.empty_like(a)
    getattr(lib(), pre + "band_bwd_first")(_p(a), a_lu, a_ld, _p(b), b_lu, b_ld, _p(part), _p(g), _p(ga), B, n, mode)
    return torch.from_numpy(ga)


def seq_band_bwd(a, a_lu, a_ld, b, b_lu, b_ld, g, mode, dtype=np.float32):
    """Both gradients the way the reference's autograd Functions obtain them
    (sparse.py:404-447, 510-545, 579-637): the first-operand kernel on (a, b), then on
    (b, a) with g (and out) transposed in band form; max mode takes the second index
    tensor from a swapped forward."""
    pre, dt = _prefix(dtype)
    out, idx, _ = seq_band_fwd(a, a_lu, a_ld, b, b_lu, b_ld, mode, dtype)
    o_lu, o_ld = a_lu + b_ld, a_ld + b_lu
    g = torch.as_tensor(_np(g, dt))
    gT = band_transpose_indexed(g, o_lu, o_ld)
    if mode == 1:
        part, partT = idx.to(g.dtype), seq_band_fwd(b, b_lu, b_ld, a, a_lu, a_ld, 1, dtype)[1].to(g.dtype)
    elif mode == 0:
        part, partT = out, band_transpose_indexed(out, o_lu, o_ld)
    else:
        part, partT = g, gT
    ga = _seq_band_bwd_first(pre, dt, a, a_lu, a_ld, b, b_lu, b_ld, part, g, mode)
    gb = _seq_band_bwd_first(pre, dt, b, b_lu, b_ld, a, a_lu, a_ld, partT, gT, mode)
    return ga, gb


def seq_band_bwdbwd(a, a_lu, a_ld, b, b_lu, b_ld, g, u, dtype=np.float32):
    """Literal quartic banded double-backward: grads of <u, grad_a> w.r.t. (a, b, g)."""
    pre, dt = _prefix(dtype)
    out, _, mx = seq_band_fwd(a, a_lu, a_ld, b, b_lu, b_ld, 0, dtype)
    a, b, g, u = _np(a, dt), _np(b, dt), _np(g, dt), _np(u, dt)
    out, mx = _np(out, dt), _np(mx, dt)
    B, n, _ = a.shape
    ga, gb, gg = np.empty_like(a), np.empty_like(b), np.empty_like(g)
    getattr(lib(), pre + "band_bwdbwd")(_p(a), a_lu, a_ld, _p(b), b_lu, b_ld, _p(g), _p(out), _p(mx), _p(u),
                                        _p(ga), _p(gb), _p(gg), B, n)
    return torch.from_numpy(ga), torch.from_numpy(gb), torch.from_numpy(gg)
