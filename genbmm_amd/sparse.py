"""Banded matrices in band storage and their semiring products.

Public surface of the reference's genbmm/sparse.py: `banddiag` (:12-30) and
`BandedMatrix` (:80-266) with `multiply`, `multiply_log`, `multiply_max`,
`transpose`, `to_dense`, `op`, `band_shift`, `band_pad`, `band_unshift`,
`col_shift`, `col_unshift`, `_expand`.

Layout: `data` is (batch, n, lu + ld + 1) and data[b, c, k] is the dense
element at row c + k - lu, column c: row c of `data` holds dense column c,
`lu` entries above the diagonal, the diagonal, `ld` entries below.

The three products run on the GPU through include/genbmm_gfx950.h
(genbmm_banded_fwd / _bwd / _bwdbwd).  The structural operations on float32
device tensors are single-pass kernels of the same library (genbmm_band_shift,
_op, _transpose, _to_dense, _from_dense), each an autograd Function whose
backward is the adjoint kernel; on host tensors (and other dtypes) they are
index arithmetic in plain torch, as in the reference.  The reference's Python
triple-loop products (`multiply_simple` and friends, :268-401), which it uses
when its extension is absent, have no counterpart here: a product on CPU
tensors raises.
"""
import operator
import os

import torch
import torch.nn.functional as F

from . import _lib

MODE_LOG, MODE_MAX, MODE_SAMPLE, MODE_MUL = 0, 1, 2, 3

# The reference sets this when its extension imports (sparse.py:3-9); here: the HIP
# library has been built.  (It selects nothing: there is no other path to fall back to.)
has_cuda = os.path.exists(_lib.LIB_PATH)


def _band_rows(n_cols, lu, ld, n_rows, device):
    """row[c, k] = c + k - lu (dense row of band cell (c, k)) and its validity mask."""
    c = torch.arange(n_cols, device=device).unsqueeze(1)
    k = torch.arange(lu + ld + 1, device=device).unsqueeze(0)
    row = c + k - lu
    return row, (row >= 0) & (row < n_rows)


def _native(t):
    """Device tensors in the library's element type take the kernels."""
    return t.is_cuda and t.dtype == torch.float32


def _struct_call(name, t, *args):
    lib = _lib.load()
    with _lib.device_of(t):
        _lib.check(getattr(lib, name)(*args, _lib.stream_of(t)), name)


class _BandShift(torch.autograd.Function):
    """out[b, c, k] = data[b, c + dcol, k + dband] or fill (genbmm_band_shift)."""

    @staticmethod
    def forward(ctx, data, w_out, dcol, dband, fill):
        data = data.contiguous()
        B, n, w_in = data.shape
        out = torch.empty(B, n, w_out, dtype=data.dtype, device=data.device)
        _struct_call("genbmm_band_shift", data, _lib.ptr(data), _lib.ptr(out), B, n, w_in, w_out,
                     dcol, dband, float(fill))
        ctx.args = (w_in, dcol, dband)
        return out

    @staticmethod
    def backward(ctx, g):
        w_in, dcol, dband = ctx.args
        return _BandShift.apply(g, w_in, -dcol, -dband, 0.0), None, None, None, None


class _BandTranspose(torch.autograd.Function):
    """Band data of the transposed matrix (genbmm_band_transpose); the adjoint is the
    transpose back."""

    @staticmethod
    def forward(ctx, data, lu, ld):
        data = data.contiguous()
        B, n, _ = data.shape
        out = torch.empty_like(data)
        _struct_call("genbmm_band_transpose", data, _lib.ptr(data), _lib.ptr(out), B, n, lu, ld)
        ctx.bands = (lu, ld)
        return out

    @staticmethod
    def backward(ctx, g):
        lu, ld = ctx.bands
        return _BandTranspose.apply(g, ld, lu), None, None


class _BandToDense(torch.autograd.Function):
    @staticmethod
    def forward(ctx, data, lu, ld, fill):
        data = data.contiguous()
        B, n, _ = data.shape
        out = torch.empty(B, n, n, dtype=data.dtype, device=data.device)
        _struct_call("genbmm_band_to_dense", data, _lib.ptr(data), _lib.ptr(out), B, n, lu, ld,
                     float(fill))
        ctx.bands = (lu, ld)
        return out

    @staticmethod
    def backward(ctx, g):
        lu, ld = ctx.bands
        return _BandFromDense.apply(g, lu, ld), None, None, None


class _BandFromDense(torch.autograd.Function):
    """Square (B, n, n) dense -> band (genbmm_band_from_dense)."""

    @staticmethod
    def forward(ctx, dense, lu, ld):
        dense = dense.contiguous()
        B, n_rows, n = dense.shape
        out = torch.empty(B, n, lu + ld + 1, dtype=dense.dtype, device=dense.device)
        _struct_call("genbmm_band_from_dense", dense, _lib.ptr(dense), _lib.ptr(out), B, n_rows, n,
                     lu, ld)
        ctx.bands = (lu, ld)
        return out

    @staticmethod
    def backward(ctx, g):
        lu, ld = ctx.bands
        return _BandToDense.apply(g, lu, ld, 0.0), None, None


# element-wise callables the library applies in one pass (others are applied by torch)
_FUSED_OPS = {torch.add: 0, operator.add: 0, torch.mul: 1, operator.mul: 1,
              torch.max: 2, torch.maximum: 2, torch.min: 3, torch.minimum: 3}


def banddiag(orig_x, lu, ld, fill=0):
    """Band storage of the dense (..., n, n) matrix `orig_x`, keeping `lu` super- and
    `ld` sub-diagonals.  Returns (band, orig_x) like the reference (sparse.py:12-30),
    whose second value is the input seen through its padded copy.  Cells that fall
    outside the matrix hold 0 (the reference ignores `fill` here as well)."""
    n_rows, n_cols = orig_x.shape[-2], orig_x.shape[-1]
    if _native(orig_x) and n_rows == n_cols and orig_x.dim() >= 3:
        flat = orig_x.reshape(-1, n_rows, n_cols)
        band = _BandFromDense.apply(flat, lu, ld)
        return band.reshape(orig_x.shape[:-2] + (n_cols, lu + ld + 1)), orig_x
    row, ok = _band_rows(n_cols, lu, ld, n_rows, orig_x.device)
    col = torch.arange(n_cols, device=orig_x.device).unsqueeze(1).expand_as(row)
    band = orig_x[..., row.clamp(0, max(n_rows - 1, 0)), col]
    band = torch.where(ok, band, torch.zeros((), dtype=band.dtype, device=band.device))
    return band, orig_x


def _band_transpose(data, lu, ld):
    """Band data of the transposed matrix (which has lu' = ld, ld' = lu):
    T[i, k] = data[i + k - ld, W - 1 - k] when that row exists, else 0
    (reference Transpose / repdiag, sparse.py:33-77)."""
    n, width = data.shape[-2], data.shape[-1]
    if _native(data) and data.dim() == 3:
        return _BandTranspose.apply(data, lu, ld)
    i = torch.arange(n, device=data.device).unsqueeze(1)
    k = torch.arange(width, device=data.device).unsqueeze(0)
    src = i + k - ld
    ok = (src >= 0) & (src < n)
    gathered = data[..., src.clamp(0, max(n - 1, 0)), (width - 1 - k).expand_as(src)]
    return torch.where(ok, gathered, torch.zeros((), dtype=data.dtype, device=data.device))


def repdiag(x, lu, ld):
    """out[..., i, j] = x[..., i + j - ld, j], 0 where that row does not exist: the
    diagonals of a band tensor re-read as rows (reference sparse.py:33-47, which pads,
    unfolds and takes a diagonal).  `repdiag(data.flip(-1), lu, ld)` is the band of the
    transposed matrix."""
    return _band_transpose(x.flip(-1), lu, ld)


class Transpose(torch.autograd.Function):
    """Band data of the transposed matrix, `Transpose.apply(val, lu, ld)` as in the
    reference (sparse.py:64-77); differentiable any number of times (the adjoint of a
    band transpose is the transpose back)."""

    @staticmethod
    def forward(ctx, val, lu, ld):
        ctx.bands = (lu, ld)
        return _band_transpose(val.detach(), lu, ld)

    @staticmethod
    def backward(ctx, grad_output):
        lu, ld = ctx.bands
        return Transpose.apply(grad_output, ld, lu), None, None


Transpose2 = Transpose  # the reference's helper for the second derivative (sparse.py:50-61)


class BandedMatrix:
    def __init__(self, data, lu, ld, fill=0):
        batch, n, off = data.shape
        assert off == lu + ld + 1, "Offsets need to add up."
        self.data = data
        self.fill = fill
        self.lu, self.ld = lu, ld
        self.width = lu + ld + 1

    # ------------------------------------------------------------ structure
    def _new(self, lu, ld):
        batch, n, _ = self.data.shape
        return self.data.new_full((batch, n, lu + ld + 1), self.fill)

    def band_shift(self, t):
        """Drop `t` leading band cells and pad `t` at the end (t < 0: the other way);
        the same numbers are re-labelled lu + t / ld - t (reference sparse.py:96-110)."""
        if t == 0:
            return self
        if _native(self.data):
            v = _BandShift.apply(self.data, self.width, 0, t, self.fill)
        elif t > 0:
            v = F.pad(self.data[:, :, t:], (0, t), value=self.fill)
        else:
            v = F.pad(self.data[:, :, :t], (-t, 0), value=self.fill)
        return BandedMatrix(v, self.lu + t, self.ld - t, self.fill)

    def band_pad(self, t):
        """Widen the band by `t` fill cells on both sides (reference sparse.py:112-123)."""
        if t == 0:
            return self
        if _native(self.data):
            v = _BandShift.apply(self.data, self.width + 2 * abs(t), 0, -abs(t), self.fill)
        else:
            v = F.pad(self.data, (abs(t), abs(t)), value=self.fill)
        return BandedMatrix(v, self.lu + t, self.ld + t, self.fill)

    def band_unshift(self):
        """One fill cell in front, last cell dropped; lu - 1 / ld + 1 (sparse.py:137-152)."""
        if _native(self.data):
            v = _BandShift.apply(self.data, self.width, 0, -1, self.fill)
        else:
            v = F.pad(self.data[:, :, :-1], (1, 0), value=self.fill)
        return BandedMatrix(v, self.lu - 1, self.ld + 1, self.fill)

    def col_shift(self, t):
        """Drop the first `t` columns and append `t` fill columns (t < 0: the other
        way); lu - t / ld + t (reference sparse.py:154-165)."""
        if t == 0:
            return self
        if _native(self.data):
            v = _BandShift.apply(self.data, self.width, t, 0, self.fill)
        elif t > 0:
            v = F.pad(self.data[:, t:, :], (0, 0, 0, t), value=self.fill)
        else:
            v = F.pad(self.data[:, :t, :], (0, 0, -t, 0), value=self.fill)
        return BandedMatrix(v, self.lu - t, self.ld + t, self.fill)

    def col_unshift(self):
        """One fill column in front, last column dropped; lu + 1 / ld - 1 (sparse.py:167-182)."""
        if _native(self.data):
            v = _BandShift.apply(self.data, self.width, -1, 0, self.fill)
        else:
            v = F.pad(self.data[:, :-1, :], (0, 0, 1, 0), value=self.fill)
        return BandedMatrix(v, self.lu + 1, self.ld - 1, self.fill)

    def to_dense(self):
        """Dense (batch, n, n) matrix; cells outside the band hold `fill` (sparse.py:184-190)."""
        batch, n, _ = self.data.shape
        if _native(self.data):
            return _BandToDense.apply(self.data, self.lu, self.ld, self.fill)
        row, ok = _band_rows(n, self.lu, self.ld, n, self.data.device)
        col = torch.arange(n, device=self.data.device).unsqueeze(1).expand_as(row)
        full = self.data.new_full((batch, n, n), self.fill)
        full[:, row[ok], col[ok]] = self.data[:, ok]
        return full

    def _expand(self, lu, ld):
        """Same matrix in a wider band (lu >= self.lu, ld >= self.ld) (sparse.py:192-197)."""
        s = lu - self.lu
        if _native(self.data):
            data = _BandShift.apply(self.data, lu + ld + 1, 0, -s, self.fill)
        else:
            data = self._new(lu, ld)
            data[:, :, s : s + self.width] = self.data
        return BandedMatrix(data, lu, ld, self.fill)

    def op(self, other, op, zero=0):
        """Element-wise `op(self, other)` on the union band; cells only one operand
        covers see `zero` for the other (reference sparse.py:199-212)."""
        lu = max(self.lu, other.lu)
        ld = max(self.ld, other.ld)
        code = _FUSED_OPS.get(op) if callable(op) and getattr(op, "__hash__", None) else None
        needs_grad = torch.is_grad_enabled() and (self.data.requires_grad or other.data.requires_grad)
        if (code is not None and not needs_grad and _native(self.data) and _native(other.data)
                and self.data.shape[:2] == other.data.shape[:2]):
            a, b = self.data.contiguous(), other.data.contiguous()
            batch, n, _ = a.shape
            data = torch.empty(batch, n, lu + ld + 1, dtype=a.dtype, device=a.device)
            _struct_call("genbmm_band_op", a, _lib.ptr(a), self.lu, self.ld, _lib.ptr(b), other.lu,
                         other.ld, _lib.ptr(data), batch, n, code, float(zero))
            return BandedMatrix(data, lu, ld, self.fill)
        data = self._new(lu, ld).fill_(zero)
        s1 = lu - self.lu
        data[:, :, s1 : s1 + self.width] = self.data
        s2 = lu - other.lu
        data[:, :, s2 : s2 + other.width] = op(data[:, :, s2 : s2 + other.width], other.data)
        return BandedMatrix(data, lu, ld, self.fill)

    def transpose(self):
        """Band form of the transposed matrix (reference sparse.py:214-218)."""
        return BandedMatrix(_band_transpose(self.data, self.lu, self.ld), self.ld, self.lu, self.fill)

    # ------------------------------------------------------------- products
    def _dense_pays(self, other, log):
        """Bands so wide that no banded kernel of the library takes them on the matrix cores (beyond
        about 225 diagonals per operand they fall to one lane per result cell, 20 to 40 times slower)
        while the matrices are small enough to multiply as dense ones: the product then goes through
        `to_dense`, the dense product on the matrix cores and `banddiag`.  Measured, forward +
        backward, 241 diagonals per operand: (+,x) 64 x 330: 0.49 ms against 7.2, 16 x 1024: 1.2 against
        9.4, 4 x 2048: 1.7 against 5.1, 4 x 4096: 11.7 against 10.5 (no longer); the log product pays
        while the result band covers a good part of the matrix - a 128 x 128 tile of the dense result
        with a cell outside the band has a cell without terms, fails the factored kernels' guard and is
        redone the exact way (64 x 330: 1.9 ms against 16.7; 16 x 512: 1.4 against 9.2; 16 x 1024: 10
        against 20; 4 x 2048: 20 against 10, no longer)."""
        a, b = self.data, other.data
        if not (_native(a) and _native(b)) or a.shape[:2] != b.shape[:2]:
            return False
        batch, n, _ = a.shape
        if min(self.width, other.width) <= 128 or batch * n * n > (1 << 28):
            return False
        if log:  # share of the dense result's cells that lie outside the result band
            lu, ld = self.lu + other.ld, self.ld + other.lu
            empty = (max(n - 1 - lu, 0) ** 2 + max(n - 1 - ld, 0) ** 2) / (2.0 * n * n)
            if empty > 0.6:
                return False
        elif n > 2048:
            return False
        return _lib.load().genbmm_banded_on_matrix_cores(self.lu, self.ld, other.lu, other.ld, batch, n) == 0

    def _product_dense(self, other, log):
        """Dense(other)^T (x) Dense(self), re-banded (reference sparse.py:229-253 in dense algebra;
        cells outside the bands are the semiring's zero, result cells outside the matrix 0)."""
        from .genmul import logbmm

        zero = -1e9 if log else 0.0       # the reference's own floor for a cell that is no term
        x = BandedMatrix(self.data, self.lu, self.ld, zero).to_dense()
        yt = BandedMatrix(other.data, other.lu, other.ld, zero).to_dense().transpose(1, 2).contiguous()
        d = logbmm(yt, x) if log else torch.bmm(yt, x)
        lu, ld = self.lu + other.ld, self.ld + other.lu
        return BandedMatrix(banddiag(d, lu, ld)[0], lu, ld, self.fill)

    def _product(self, other, fn):
        batch, n, _ = self.data.shape
        assert other.data.shape[1] == n
        lu = self.lu + other.ld
        ld = self.ld + other.lu
        if (fn is bandedbmm or fn is bandedlogbmm) and self._dense_pays(other, fn is bandedlogbmm):
            return self._product_dense(other, fn is bandedlogbmm)
        # views are copied here, by a differentiable torch operation, so that the
        # Functions save (and differentiate with respect to) what they were given
        # (float16 / bfloat16 bands go to the `_f16` / `_bf16` entry points as they are)
        a, b = self.data, other.data
        out = fn(a.contiguous(), self.lu, self.ld, b.contiguous(), other.lu, other.ld, lu, ld)
        return BandedMatrix(out, lu, ld, self.fill)

    def multiply(self, other):
        """Dense(other)^T @ Dense(self) in band form (reference sparse.py:229-240)."""
        return self._product(other, bandedbmm)

    def multiply_log(self, other):
        """The same product in the (logsumexp, +) semiring (reference sparse.py:242-253)."""
        return self._product(other, bandedlogbmm)

    def multiply_max(self, other):
        """The same product in the (max, +) semiring (reference sparse.py:255-266)."""
        return self._product(other, bandedmaxbmm)

    def multiply_sample(self, other, stream=None):
        """The log product whose gradient is a one-hot sample: every result cell draws one of
        its terms k with probability exp(a + b - out) and hands its incoming gradient to that
        term's two cells, as `samplebmm` does for dense operands.  The reference's band kernel
        stops at the log, max and (+, *) products (banded_cuda_kernel.cu:42, 65, 76); this is
        its dense sampling rule (matmul_cuda_kernel.cu:107-118) on a band cell's terms.
        `stream` = (seed, offset) pins the Philox stream; None follows torch's CUDA generator."""
        return self._product(other, lambda *args: BandedSampleMul.apply(*args, stream))

    def multiply_back(self, other, out, grad_out):
        """Gradient of `self.multiply(other)` with respect to self, given the gradient of
        the product's band tensor (reference sparse.py:363-379; `out` is not needed)."""
        a, b = self.data.detach().contiguous(), other.data.detach().contiguous()
        g = grad_out.data if isinstance(grad_out, BandedMatrix) else grad_out
        grad_a, _ = _backward(a, b, (self.lu, self.ld, other.lu, other.ld), None, None, g, MODE_MUL)
        return BandedMatrix(grad_a, self.lu, self.ld, self.fill)


# ------------------------------------------------------------------ autograd
def _f64(t):
    return t.dtype == torch.float64


def _sfx(t):
    """Entry-point suffix for the tensor's element type ("", "_f16", "_bf16")."""
    return _lib.HALF_SUFFIX.get(t.dtype, "")


def _check_pair(a, b):
    dtype = torch.float32
    if isinstance(a, torch.Tensor) and (_f64(a) or a.dtype in _lib.HALF_SUFFIX):
        dtype = a.dtype
    _lib.require(a, "a", dtype=dtype)
    _lib.require(b, "b", dtype=dtype, device=a.device)
    if a.shape[:2] != b.shape[:2]:
        raise RuntimeError("banded operands disagree: %s vs %s" % (tuple(a.shape), tuple(b.shape)))
    return a.shape[0], a.shape[1]


def _call(name, t, *args):
    lib = _lib.load()
    with _lib.device_of(t):
        _lib.check(getattr(lib, name)(*args, _lib.stream_of(t)), name)


def _forward(a, a_lu, a_ld, b, b_lu, b_ld, mode):
    a = a.contiguous()
    b = b.contiguous()
    B, n = _check_pair(a, b)
    if a.shape[2] != a_lu + a_ld + 1 or b.shape[2] != b_lu + b_ld + 1:
        raise RuntimeError("band widths do not match lu + ld + 1")
    wo = a.shape[2] + b.shape[2] - 1
    out = torch.empty(B, n, wo, dtype=a.dtype, device=a.device)
    idx = torch.empty(B, n, wo, dtype=torch.int32, device=a.device) if mode == MODE_MAX else None
    if _f64(a):  # the double-precision entry points take no workspace
        _call("genbmm_banded_fwd_f64", a, _lib.ptr(a), a_lu, a_ld, _lib.ptr(b), b_lu, b_ld,
              _lib.ptr(out), _lib.ptr(idx), B, n, mode)
        return a, b, out, (None if mode == MODE_LOG else idx)
    # log product: the library's workspace (exp(a - max), exp(b - max), maxima, 1/sum),
    # which stands where the reference's `maxes` stands
    ws = None
    if mode == MODE_LOG:
        size = _lib.load().genbmm_banded_workspace_size(a_lu, a_ld, b_lu, b_ld, B, n)
        ws = torch.empty(size, dtype=torch.float32, device=a.device)
    _call("genbmm_banded_fwd" + _sfx(a), a, _lib.ptr(a), a_lu, a_ld, _lib.ptr(b), b_lu, b_ld,
          _lib.ptr(out), _lib.ptr(idx), _lib.ptr(ws), B, n, mode)
    return a, b, out, (ws if mode == MODE_LOG else idx)


def _backward(a, b, bands, out, idx, g, mode, ws=None):
    a_lu, a_ld, b_lu, b_ld = bands
    B, n = a.shape[0], a.shape[1]
    g = g.to(a.dtype).contiguous()
    grad_a = torch.empty_like(a)
    grad_b = torch.empty_like(b)
    if _f64(a):
        _call("genbmm_banded_bwd_f64", a, _lib.ptr(a), a_lu, a_ld, _lib.ptr(b), b_lu, b_ld,
              _lib.ptr(out), _lib.ptr(idx), _lib.ptr(g), _lib.ptr(grad_a), _lib.ptr(grad_b), B, n, mode)
        return grad_a, grad_b
    # g / sum per output cell, which both gradients of the log product share, goes to a
    # buffer of this call's own: the forward's workspace stays as the forward left it, so
    # backward passes over one forward may overlap (other streams, retained graphs)
    scratch = None
    if mode == MODE_LOG and ws is not None:
        need = _lib.load().genbmm_banded_scratch_size(a_lu, a_ld, b_lu, b_ld, B, n)
        scratch = torch.empty(need, dtype=torch.float32, device=a.device) if need else None
    _call("genbmm_banded_bwd_scratch" + _sfx(a), a, _lib.ptr(a), a_lu, a_ld, _lib.ptr(b), b_lu, b_ld,
          _lib.ptr(out), _lib.ptr(idx), _lib.ptr(ws), _lib.ptr(scratch), _lib.ptr(g), _lib.ptr(grad_a),
          _lib.ptr(grad_b), B, n, mode)
    return grad_a, grad_b


_NO_BAND_GRADS = (None,) * 6


class BandedMul(torch.autograd.Function):
    """(+, *) banded product (reference sparse.py:404-447)."""

    @staticmethod
    def forward(ctx, a, a_lu, a_ld, b, b_lu, b_ld, o_lu, o_ld):
        _, _, out, _ = _forward(a, a_lu, a_ld, b, b_lu, b_ld, MODE_MUL)
        ctx.save_for_backward(a, b)
        ctx.bands = (a_lu, a_ld, b_lu, b_ld)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        a, b = (t.contiguous() for t in ctx.saved_tensors)
        grad_a, grad_b = _backward(a, b, ctx.bands, None, None, grad_output, MODE_MUL)
        return (grad_a, None, None, grad_b) + (None,) * 4


class _BandedLogGrad(torch.autograd.Function):
    """(a, b, g, out) -> (grad_a, grad_b) of the log product, differentiable in
    (a, b, g).  Plays the role of the reference's BandedLogMulBack
    (sparse.py:466-508), which yields one gradient per call and needs g, out and
    maxes transposed in band form for the second operand."""

    @staticmethod
    def forward(ctx, a, b, g, out, ws, bands):
        grad_a, grad_b = _backward(a, b, bands, out, None, g, MODE_LOG, ws)
        ctx.save_for_backward(a, b, g, out)
        ctx.bands = bands
        ctx.set_materialize_grads(False)
        return grad_a, grad_b

    @staticmethod
    def backward(ctx, u_a, u_b):
        if u_a is None and u_b is None:
            return (None,) * 6
        a, b, g, out = ctx.saved_tensors
        a_lu, a_ld, b_lu, b_ld = ctx.bands
        u_a = None if u_a is None else u_a.contiguous()
        u_b = None if u_b is None else u_b.contiguous()
        ga, gb, gg = torch.empty_like(a), torch.empty_like(b), torch.empty_like(g)
        if a.dtype in _lib.HALF_SUFFIX:
            # the gradient with respect to g is read back by the other two: a float copy of it
            t = torch.empty(g.shape, dtype=torch.float32, device=g.device)
            _call("genbmm_banded_bwdbwd" + _sfx(a), a, _lib.ptr(a), a_lu, a_ld, _lib.ptr(b), b_lu, b_ld,
                  _lib.ptr(out), _lib.ptr(g), _lib.ptr(u_a), _lib.ptr(u_b), _lib.ptr(ga), _lib.ptr(gb),
                  _lib.ptr(gg), _lib.ptr(t), a.shape[0], a.shape[1])
            return ga, gb, gg, None, None, None
        _call("genbmm_banded_bwdbwd_f64" if _f64(a) else "genbmm_banded_bwdbwd", a, _lib.ptr(a),
              a_lu, a_ld, _lib.ptr(b), b_lu, b_ld, _lib.ptr(out), _lib.ptr(g), _lib.ptr(u_a), _lib.ptr(u_b),
              _lib.ptr(ga), _lib.ptr(gb), _lib.ptr(gg), a.shape[0], a.shape[1])
        return ga, gb, gg, None, None, None


class BandedLogMul(torch.autograd.Function):
    """(logsumexp, +) banded product, twice differentiable (reference sparse.py:510-545)."""

    @staticmethod
    def forward(ctx, a, a_lu, a_ld, b, b_lu, b_ld, o_lu, o_ld):
        _, _, out, ws = _forward(a, a_lu, a_ld, b, b_lu, b_ld, MODE_LOG)
        # the operands as given (the reference does the same, sparse.py:510-520): when they
        # are views, the copies are taken in backward, where autograd records them, so
        # that second-order gradients flow to the caller's tensors
        ctx.save_for_backward(a, b, out, ws)
        ctx.bands = (a_lu, a_ld, b_lu, b_ld)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        a, b, out, ws = ctx.saved_tensors
        a, b = a.contiguous(), b.contiguous()
        g = grad_output.to(a.dtype).contiguous()
        grad_a, grad_b = _BandedLogGrad.apply(a, b, g, out, ws, ctx.bands)
        return (grad_a, None, None, grad_b) + (None,) * 4


class BandedMaxMul(torch.autograd.Function):
    """(max, +) banded product (reference sparse.py:579-637).  One forward launch:
    the arg-max is kept in a's band frame and both gradients read it there, where the
    reference runs the forward a second time with the operands swapped."""

    @staticmethod
    def forward(ctx, a, a_lu, a_ld, b, b_lu, b_ld, o_lu, o_ld):
        _, _, out, idx = _forward(a, a_lu, a_ld, b, b_lu, b_ld, MODE_MAX)
        ctx.save_for_backward(a, b, idx)
        ctx.bands = (a_lu, a_ld, b_lu, b_ld)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        a, b, idx = ctx.saved_tensors
        a, b = a.contiguous(), b.contiguous()
        grad_a, grad_b = _backward(a, b, ctx.bands, None, idx, grad_output, MODE_MAX)
        return (grad_a, None, None, grad_b) + (None,) * 4


class BandedSampleMul(torch.autograd.Function):
    """Banded sample product (`BandedMatrix.multiply_sample`): the log product forward, the
    arg-max scatter of the drawn indices backward - the banded form of the reference's
    SampleMatMul (genmul.py:68-81)."""

    @staticmethod
    def forward(ctx, a, a_lu, a_ld, b, b_lu, b_ld, o_lu, o_ld, stream=None):
        from .genmul import _next_stream

        a, b = a.contiguous(), b.contiguous()
        B, n = _check_pair(a, b)
        if a.shape[2] != a_lu + a_ld + 1 or b.shape[2] != b_lu + b_ld + 1:
            raise RuntimeError("band widths do not match lu + ld + 1")
        seed, offset = _next_stream(a.device) if stream is None else stream
        seed, offset = int(seed) & 0xFFFFFFFFFFFFFFFF, int(offset) & 0xFFFFFFFFFFFFFFFF
        wo = a.shape[2] + b.shape[2] - 1
        out = torch.empty(B, n, wo, dtype=a.dtype, device=a.device)
        idx = torch.empty(B, n, wo, dtype=torch.int32, device=a.device)
        if _f64(a):
            _call("genbmm_banded_sample_fwd_f64", a, _lib.ptr(a), a_lu, a_ld, _lib.ptr(b), b_lu, b_ld,
                  _lib.ptr(out), _lib.ptr(idx), seed, offset, B, n)
        else:
            size = _lib.load().genbmm_banded_workspace_size(a_lu, a_ld, b_lu, b_ld, B, n)
            ws = torch.empty(size, dtype=torch.float32, device=a.device)
            _call("genbmm_banded_sample_fwd" + _sfx(a), a, _lib.ptr(a), a_lu, a_ld, _lib.ptr(b), b_lu, b_ld,
                  _lib.ptr(out), _lib.ptr(idx), _lib.ptr(ws), seed, offset, B, n)
        ctx.save_for_backward(a, b, idx)
        ctx.bands = (a_lu, a_ld, b_lu, b_ld)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        a, b, idx = ctx.saved_tensors
        grad_a, grad_b = _backward(a, b, ctx.bands, None, idx, grad_output, MODE_SAMPLE)
        return (grad_a, None, None, grad_b) + (None,) * 5


bandedbmm = BandedMul.apply
bandedlogbmm = BandedLogMul.apply
bandedmaxbmm = BandedMaxMul.apply
