"""Dense semiring batched matmul with autograd: logbmm, maxbmm, samplebmm, prodmaxbmm.

Same public contract as the reference's genbmm/genmul.py:100-103: each op takes
contiguous device tensors a (B, M, K) and b (B, K, N) and returns (B, M, N);
all four are differentiable and logbmm is twice differentiable.  The work is
done by the HIP kernels behind the C ABI in include/genbmm_gfx950.h.

Differences in mechanism (not in results):
  * logbmm's backward produces grad_a and grad_b from one library call that
    reads every operand in place; the reference calls its kernel twice and
    transposes b, a, g, out, maxes and the result in between (genmul.py:35-41).
  * instead of the (B, M, N) `maxes` tensor the forward saves a workspace sized by
    the library: row maxima of a, column maxima of b and a few per-tile flags,
    which let forward and backward factor exp(a + b) wherever that is exact
    (csrc/logbmm.hip), and - for shapes that run on the matrix cores - the
    factors exp(a - max), exp(b - max) and 1/sum, so that the backward takes no
    exponential at all (csrc/logbmm_mfma.h).
  * the arg-max / sample index stays int32 into the backward; the reference
    converts it (and a, b, g) to float first (genmul.py:62-65).
  * samplebmm draws its uniforms from a counter-based Philox4x32-10 stream
    keyed by torch's CUDA generator seed instead of torch::rand
    (matmul_cuda_kernel.cu:517).

Element types: float32 takes the kernels above; float64 takes the library's
double-precision entry points (`*_f64`, no workspaces); float16 / bfloat16 take the
same kernels compiled for that element type (`*_f16` / `*_bf16`: the loads widen,
arithmetic and workspaces are float32, the stores round to nearest), the reference's
AT_DISPATCH_FLOATING_TYPES_AND_HALF (matmul_cuda_kernel.cu:489).  Only logbmm's
double backward widens half tensors on the host.

Beyond the reference's contract the four functions also take operands with any
number of leading batch dimensions (equal or broadcastable; they are flattened to
one and restored on the result) and non-contiguous operands (made contiguous;
the reference raises).  Both conversions happen
outside the autograd Functions with differentiable torch operations, so first-
and second-order gradients reach the tensors the caller passed.  CPU tensors
raise RuntimeError, as in the reference (matmul_cuda.cpp:65-67).
"""
import torch

from . import _lib

_COMPUTE = torch.float32   # every workspace, whatever the tensors' element type
_DTYPES = (torch.float32, torch.float64, torch.float16, torch.bfloat16)


def _f64(t):
    return t.dtype == torch.float64


def _sfx(t):
    """Suffix of the entry points for t's element type ('' for float32)."""
    return _lib.HALF_SUFFIX.get(t.dtype, "")


PATH_AUTO, PATH_EXACT, PATH_VALU, PATH_FACTORS, PATH_MFMA32 = 0, 1, 2, 3, 4  # GENBMM_PATH_* of the C header


def _prep(a, b):
    """Checks in front of the library for operands that are already in its form
    (3-D, contiguous, float32 or float64, on one device)."""
    if not isinstance(a, torch.Tensor) or not isinstance(b, torch.Tensor):
        raise RuntimeError("a and b must be tensors")
    if a.dtype != b.dtype:
        raise RuntimeError("a and b must have the same dtype, got %s and %s" % (a.dtype, b.dtype))
    if a.dtype not in _DTYPES:
        raise RuntimeError(
            "genbmm_amd takes float32, float64, float16 or bfloat16 tensors; %s is not supported" % a.dtype
        )
    return _lib.dense_dims(a, b)


def _canonical(a, b):
    """(a3, b3, restore): the operands as contiguous 3-D tensors and the function that
    gives the (B, M, N) result the caller's batch shape.
    Everything done here is an ordinary differentiable torch operation."""
    if not isinstance(a, torch.Tensor) or not isinstance(b, torch.Tensor):
        raise RuntimeError("a and b must be tensors")
    if not a.is_cuda or not b.is_cuda:
        raise RuntimeError("a and b must be CUDA tensors")
    if a.dtype != b.dtype:
        raise RuntimeError("a and b must have the same dtype, got %s and %s" % (a.dtype, b.dtype))
    if a.dim() < 2 or b.dim() < 2:
        raise RuntimeError("a and b must have at least 2 dimensions")
    if a.shape[-1] != b.shape[-2]:
        raise RuntimeError("shape mismatch: a is %s, b is %s" % (tuple(a.shape), tuple(b.shape)))
    if a.dtype not in _DTYPES:
        raise RuntimeError(
            "genbmm_amd takes float32, float64, float16 or bfloat16 tensors; %s is not supported" % a.dtype
        )
    batch = None
    if a.dim() != 3 or b.dim() != 3 or a.shape[0] != b.shape[0]:
        try:
            batch = torch.broadcast_shapes(a.shape[:-2], b.shape[:-2])
        except RuntimeError:
            raise RuntimeError("shape mismatch: a is %s, b is %s" % (tuple(a.shape), tuple(b.shape)))
        a = a.expand(batch + a.shape[-2:]).reshape((-1,) + a.shape[-2:])
        b = b.expand(batch + b.shape[-2:]).reshape((-1,) + b.shape[-2:])
    a, b = a.contiguous(), b.contiguous()

    def restore(out):
        if batch is not None:
            out = out.reshape(batch + out.shape[-2:])
        return out

    return a, b, restore


def _call(name, t, *args):
    lib = _lib.load()
    with _lib.device_of(t):
        _lib.check(getattr(lib, name)(*args, _lib.stream_of(t)), name)


# --------------------------------------------------------------------- logbmm
class _LogBmmGrad(torch.autograd.Function):
    """(a, b, g, out) -> (grad_a, grad_b); itself differentiable in (a, b, g).

    Plays the role of the reference's LogMatMulBack (genmul.py:11-24), which
    yields grad_a only and is applied twice per backward.
    """

    @staticmethod
    def forward(ctx, a, b, g, out, stats, path):
        B, M, K, N = _lib.dense_dims(a, b)
        grad_a = torch.empty_like(a)
        grad_b = torch.empty_like(b)
        if _f64(a):
            _call("genbmm_logbmm_bwd_f64", a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(g),
                  _lib.ptr(grad_a), _lib.ptr(grad_b), B, M, K, N)
        else:
            _call("genbmm_logbmm_bwd_path" + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(g),
                  _lib.ptr(stats), _lib.ptr(grad_a), _lib.ptr(grad_b), B, M, K, N, path)
        ctx.save_for_backward(a, b, g, out)
        ctx.set_materialize_grads(False)
        return grad_a, grad_b

    @staticmethod
    def backward(ctx, u_a, u_b):
        if u_a is None and u_b is None:
            return None, None, None, None, None, None
        a, b, g, out = ctx.saved_tensors
        B, M, K, N = _lib.dense_dims(a, b)
        u_a = None if u_a is None else u_a.to(a.dtype).contiguous()
        u_b = None if u_b is None else u_b.to(a.dtype).contiguous()
        ga = torch.empty_like(a)
        gb = torch.empty_like(b)
        gg = torch.empty_like(g)
        if _f64(a):
            _call("genbmm_logbmm_bwdbwd_f64", a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(g),
                  _lib.ptr(u_a), _lib.ptr(u_b), _lib.ptr(ga), _lib.ptr(gb), _lib.ptr(gg), B, M, K, N)
        else:
            # scratch for the factored form on the matrix cores (and, for float16 / bfloat16 tensors, where
            # the gradient with respect to g stays unrounded for the other two gradients)
            ws = torch.empty(_lib.load().genbmm_logbmm_bwdbwd_ws_size(B, M, K, N), dtype=_COMPUTE, device=a.device)
            _call("genbmm_logbmm_bwdbwd_ws" + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(g),
                  _lib.ptr(u_a), _lib.ptr(u_b), _lib.ptr(ga), _lib.ptr(gb), _lib.ptr(gg), _lib.ptr(ws), B, M, K, N)
        return ga, gb, gg, None, None, None


class LogMatMul(torch.autograd.Function):
    """out[b,m,n] = logsumexp_k(a[b,m,k] + b[b,k,n])   (reference genmul.py:27-41).
    `path` names the library's kernel family (PATH_AUTO unless a test says otherwise)."""

    @staticmethod
    def forward(ctx, a, b, path=PATH_AUTO):
        B, M, K, N = _prep(a, b)
        out = torch.empty(B, M, N, dtype=a.dtype, device=a.device)
        if _f64(a):
            stats = a.new_empty(0)
            _call("genbmm_logbmm_fwd_f64", a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), B, M, K, N)
        else:
            # the library's workspace: what the reference's `maxes` becomes
            stats = torch.empty(_lib.load().genbmm_logbmm_stats_size_path(B, M, K, N, path), dtype=_COMPUTE,
                                device=a.device)
            _call("genbmm_logbmm_fwd_path" + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out),
                  _lib.ptr(stats), B, M, K, N, path)
        ctx.save_for_backward(a, b, out, stats)
        ctx.path = path
        return out

    @staticmethod
    def backward(ctx, grad_output):
        a, b, out, stats = ctx.saved_tensors
        grad_a, grad_b = _LogBmmGrad.apply(a, b, grad_output.to(a.dtype).contiguous(), out, stats, ctx.path)
        return grad_a, grad_b, None


# ------------------------------------------------- max / sample / prod-max
def _argmax_backward(ctx, grad_output, prod):
    ct = ctx.compute
    if prod:
        idx, factors, a, b = ctx.saved_tensors
    else:
        (idx,) = ctx.saved_tensors
    B, M, K, N = ctx.dims
    g = grad_output.to(ct).contiguous()
    grad_a = torch.empty(B, M, K, dtype=ct, device=g.device)
    grad_b = torch.empty(B, K, N, dtype=ct, device=g.device)
    if ct == torch.float64:
        if prod:
            _call("genbmm_prodmax_bwd_f64", g, _lib.ptr(a), _lib.ptr(b), _lib.ptr(idx), _lib.ptr(g),
                  _lib.ptr(grad_a), _lib.ptr(grad_b), B, M, K, N)
        else:
            _call("genbmm_argmax_bwd_f64", g, _lib.ptr(idx), _lib.ptr(g), _lib.ptr(grad_a),
                  _lib.ptr(grad_b), B, M, K, N)
    elif prod:
        # the factors a[m, idx], b[idx, n] were stored by the forward: a and b are not read
        _call("genbmm_prodmax_bwd" + _sfx(g), g, _lib.ptr(None), _lib.ptr(None), _lib.ptr(idx),
              _lib.ptr(factors), _lib.ptr(g), _lib.ptr(grad_a), _lib.ptr(grad_b), B, M, K, N)
    else:
        _call("genbmm_argmax_bwd" + _sfx(g), g, _lib.ptr(idx), _lib.ptr(g), _lib.ptr(grad_a),
              _lib.ptr(grad_b), B, M, K, N)
    return grad_a, grad_b


def _max_forward(a, b, prod, factors=None):
    """(out, idx) of the max / prod-max product through the library; `factors` (2, B, M, N) receives
    a[m, idx], b[idx, n] of prod-max.  A long reduction over few output tiles is cut into S pieces
    of K, each a batch item of its own (see _reduction_splits): the pieces' maxima are joined
    here - the first piece that attains the maximum wins, as the lowest k does inside a piece -
    and the indices become indices into the whole of K."""
    B, M, K = a.shape
    N = b.shape[2]
    S = 1 if _f64(a) else _reduction_splits(B, M, K, N)
    if S > 1 and a.dtype == torch.float32 and _lib.load().genbmm_maxbmm_fwd_pieces(B, M, K, N) > 1:
        S = 1       # the library cuts the reduction axis of this problem itself
    name = "genbmm_prodmaxbmm_fwd" if prod else "genbmm_maxbmm_fwd"
    if S == 1:
        out = torch.empty(B, M, N, dtype=a.dtype, device=a.device)
        idx = torch.empty(B, M, N, dtype=torch.int32, device=a.device)
        if _f64(a):
            _call(name + "_f64", a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(idx), B, M, K, N)
        elif prod:
            _call(name + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(idx), _lib.ptr(factors), B, M, K, N)
        else:
            _call(name + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(idx), B, M, K, N)
        return out, idx
    Ks = K // S
    # (float16 / bfloat16 operands: the pieces are compared unrounded, in float32 - two pieces whose
    # maxima round to the same half value must still be told apart - and the result is rounded once)
    wide_a = a.float() if a.dtype in _lib.HALF_SUFFIX else a
    wide_b = b.float() if b.dtype in _lib.HALF_SUFFIX else b
    a_s = wide_a.view(B, M, S, Ks).transpose(1, 2).reshape(B * S, M, Ks).contiguous()
    b_s = wide_b.view(B * S, Ks, N)
    vals = torch.empty(B * S, M, N, dtype=a_s.dtype, device=a.device)
    idxs = torch.empty(B * S, M, N, dtype=torch.int32, device=a.device)
    if prod:
        fac_s = torch.empty(2, B * S, M, N, dtype=_COMPUTE, device=a.device)
        _call(name, a, _lib.ptr(a_s), _lib.ptr(b_s), _lib.ptr(vals), _lib.ptr(idxs), _lib.ptr(fac_s), B * S, M, Ks, N)
    else:
        _call(name, a, _lib.ptr(a_s), _lib.ptr(b_s), _lib.ptr(vals), _lib.ptr(idxs), B * S, M, Ks, N)
    vals, idxs = vals.view(B, S, M, N), idxs.view(B, S, M, N)
    # a piece without a term above the -1e9 floor reports the floor and index -1: it never wins
    # against a piece with one, and if no piece has one the result is the floor and -1 as well
    top = vals.amax(1, keepdim=True)
    pieces = torch.arange(S, device=a.device).view(1, S, 1, 1)
    first = torch.where(vals == top, pieces, torch.full_like(pieces, S)).amin(1, keepdim=True)   # lowest piece on ties
    first = first.clamp(max=S - 1)      # (all NaN: cannot happen, NaN terms never win inside a piece)
    out = torch.gather(vals, 1, first).squeeze(1)
    local = torch.gather(idxs, 1, first).squeeze(1)
    idx = torch.where(local >= 0, local + (first.squeeze(1) * Ks).to(torch.int32), local).contiguous()
    if prod:
        fac = fac_s.view(2, B, S, M, N)
        factors.copy_(torch.gather(fac, 2, first.unsqueeze(0).expand(2, -1, -1, -1, -1)).squeeze(2))
    return out.to(a.dtype).contiguous(), idx


class MaxMatMul(torch.autograd.Function):
    """out = max_k(a + b), ties to the lowest k   (reference genmul.py:52-65)."""

    @staticmethod
    def forward(ctx, a, b):
        dims = _prep(a, b)
        out, idx = _max_forward(a, b, False)
        ctx.save_for_backward(idx)
        ctx.dims, ctx.compute = dims, a.dtype
        return out

    @staticmethod
    def backward(ctx, grad_output):
        return _argmax_backward(ctx, grad_output, prod=False)


class ProdMaxMatMul(torch.autograd.Function):
    """out = max_k(a * b)   (reference genmul.py:84-97)."""

    @staticmethod
    def forward(ctx, a, b):
        dims = _prep(a, b)
        B, M, K, N = dims
        empty = a.new_empty(0)
        if _f64(a):
            out, idx = _max_forward(a, b, True)
            ctx.save_for_backward(idx, empty, a, b)
        else:
            factors = torch.empty(2, B, M, N, dtype=_COMPUTE, device=a.device)
            out, idx = _max_forward(a, b, True, factors)
            ctx.save_for_backward(idx, factors, empty, empty)
        ctx.dims, ctx.compute = dims, a.dtype
        return out

    @staticmethod
    def backward(ctx, grad_output):
        return _argmax_backward(ctx, grad_output, prod=True)


_SEED_SALT = 0x67656E626D6D  # keeps the stream apart from torch's own Philox use


def _next_stream(device):
    """(seed, offset) for the next samplebmm call: follows torch.manual_seed and
    advances the CUDA generator's offset so that successive calls differ."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    gen = torch.cuda.default_generators[index]
    seed = (gen.initial_seed() ^ _SEED_SALT) & 0xFFFFFFFFFFFFFFFF
    offset = gen.get_offset()
    gen.set_offset(offset + 4)
    return seed, offset


class SampleMatMul(torch.autograd.Function):
    """out = logsumexp_k(a + b); the gradient is a one-hot sample k ~ softmax_k(a + b)
    (reference genmul.py:68-81).  `stream` = (seed, offset) pins the Philox stream."""

    @staticmethod
    def forward(ctx, a, b, stream=None):
        dims = _prep(a, b)
        B, M, K, N = dims
        seed, offset = _next_stream(a.device) if stream is None else stream
        out = torch.empty(B, M, N, dtype=a.dtype, device=a.device)
        idx = torch.empty(B, M, N, dtype=torch.int32, device=a.device)
        seed, offset = int(seed) & 0xFFFFFFFFFFFFFFFF, int(offset) & 0xFFFFFFFFFFFFFFFF
        if _f64(a):
            _call("genbmm_samplebmm_fwd_f64", a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out),
                  _lib.ptr(idx), seed, offset, B, M, K, N)
        else:
            stats = torch.empty(_lib.load().genbmm_samplebmm_stats_size(B, M, K, N), dtype=_COMPUTE,
                                device=a.device)
            _call("genbmm_samplebmm_fwd" + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(idx),
                  _lib.ptr(stats), seed, offset, B, M, K, N)
        ctx.save_for_backward(idx)
        ctx.dims, ctx.compute = dims, a.dtype
        return out

    @staticmethod
    def backward(ctx, grad_output):
        return _argmax_backward(ctx, grad_output, prod=False) + (None,)


def _reduction_splits(B, M, K, N):
    """How many pieces to cut the reduction axis into.  The kernels give every output tile to one
    workgroup that walks all of K: a problem with few tiles and a long K would run on a few
    of the 256 compute units.  Such a problem is cut into S pieces of K (S divides K), each a
    batch item of its own; the pieces are joined by a logsumexp over S."""
    tiles = B * ((M + 127) // 128) * ((N + 127) // 128)
    # (from K = 4096 on: below, the extra launches of the split cost what it saves)
    if tiles >= 128 or K < 4096 or M * N == 0:
        return 1
    want = min(K // 256, (255 + tiles) // tiles)
    for s in range(want, 1, -1):
        if K % s == 0:
            return s
    return 1


def logbmm(a, b):
    """genbmm.logbmm(a, b): out[..., m, n] = logsumexp_k(a[..., m, k] + b[..., k, n])."""
    a, b, restore = _canonical(a, b)
    B, M, K = a.shape
    N = b.shape[2]
    S = 1 if _f64(a) else _reduction_splits(B, M, K, N)
    if S > 1 and _lib.load().genbmm_logbmm_fwd_pieces(B, M, K, N) > 1:
        # the library's forward cuts the reduction axis of this problem itself (float16 / bfloat16
        # operands: the float function on the widened tensors, rounded once)
        if a.dtype in _lib.HALF_SUFFIX:
            return restore(LogMatMul.apply(a.float(), b.float(), PATH_AUTO).to(a.dtype))
        S = 1
    if S > 1:  # differentiable torch operations around the same kernels (any order of derivative)
        # float16 / bfloat16 operands: the pieces are formed and joined in float32 and the result is
        # rounded once, as the unsplit kernels do (a piece stored in the half type would round twice)
        wide = a.float() if a.dtype in _lib.HALF_SUFFIX else a
        a_s = wide.view(B, M, S, K // S).transpose(1, 2).reshape(B * S, M, K // S).contiguous()
        b_s = (b.float() if b.dtype in _lib.HALF_SUFFIX else b).view(B * S, K // S, N)
        parts = LogMatMul.apply(a_s, b_s, PATH_AUTO).view(B, S, M, N)
        return restore(torch.logsumexp(parts, dim=1).to(a.dtype))
    # float16 / bfloat16 tensors keep 1 / sum in float32 for the backward (PATH_FACTORS): with the
    # maxima alone it would be rebuilt from `out` as stored, i.e. rounded to 11 or 8 bits
    return restore(LogMatMul.apply(a, b, PATH_FACTORS if a.dtype in _lib.HALF_SUFFIX else PATH_AUTO))


def logbmm_on_path(a, b, path):
    """logbmm with the library's kernel family named (PATH_AUTO / PATH_EXACT / PATH_VALU / PATH_FACTORS:
    as PATH_AUTO, but autograd saves exp(a - max), exp(b - max) and 1 / sum beside the maxima - three
    more tensors than the reference saves - and the matrix-core backward takes no exponential /
    PATH_MFMA32: as PATH_AUTO with the fp32 matrix instruction for every tiled shape);
    forward and backward both use it.  For tests and measurements."""
    a, b, restore = _canonical(a, b)
    return restore(LogMatMul.apply(a, b, path))


def maxbmm(a, b):
    """genbmm.maxbmm(a, b): max_k(a + b); the gradient goes to the lowest arg-max."""
    a, b, restore = _canonical(a, b)
    return restore(MaxMatMul.apply(a, b))


def prodmaxbmm(a, b):
    """genbmm.prodmaxbmm(a, b): max_k(a * b)."""
    a, b, restore = _canonical(a, b)
    return restore(ProdMaxMatMul.apply(a, b))


def samplebmm(a, b, stream=None):
    """genbmm.samplebmm(a, b); `stream=(seed, offset)` makes the draw reproducible."""
    a, b, restore = _canonical(a, b)
    return restore(SampleMatMul.apply(a, b, stream))
