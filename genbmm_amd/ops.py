"""The dense and banded products as `torch.library` custom operators (float32; the dense
ones also float16 / bfloat16).

`genbmm_amd.logbmm` and friends are `torch.autograd.Function`s, which `torch.compile`
cannot trace through.  This module registers the same library calls as operators of the
`genbmm_amd::` namespace, each with a shape-only ("fake") implementation and a backward
formula written in terms of further operators, so that graphs containing them can be
captured (`torch.compile(..., fullgraph=True)`, `torch.export`) and differentiated - twice
for logbmm.  The reference has no counterpart: its extension is reached through
autograd Functions only (genbmm/genmul.py).

    from genbmm_amd import ops
    y = ops.logbmm(a, b)          # also ops.maxbmm, ops.prodmaxbmm, ops.samplebmm
    c = ops.banded_multiply_log(a_band, a_lu, a_ld, b_band, b_lu, b_ld)   # also banded_multiply, _max

The arithmetic is that of genmul.py's Functions: the same C-ABI entry points with the
same workspaces.
"""
from typing import Tuple

import torch
from torch import Tensor

from . import _lib

_F32 = torch.float32


def _dims(a: Tensor, b: Tensor):
    B, M, K = a.shape
    return B, M, K, b.shape[2]


def _check(a: Tensor, b: Tensor):
    if a.dtype != b.dtype or (a.dtype != _F32 and a.dtype not in _lib.HALF_SUFFIX):
        raise RuntimeError("genbmm_amd.ops: float32, float16 or bfloat16 tensors of one type "
                           "(use genbmm_amd.logbmm etc. for others)")
    return _lib.dense_dims(a, b)


def _sfx(t: Tensor):
    """Suffix of the library's entry points for t's element type."""
    return _lib.HALF_SUFFIX.get(t.dtype, "")


def _call(name, t, *args):
    lib = _lib.load()
    with _lib.device_of(t):
        _lib.check(getattr(lib, name)(*args, _lib.stream_of(t)), name)


def _stats_size(B, M, K, N):
    return int(_lib.load().genbmm_logbmm_stats_size(int(B), int(M), int(K), int(N)))


# ------------------------------------------------------------------------ logbmm
@torch.library.custom_op("genbmm_amd::logbmm_fwd", mutates_args=())
def logbmm_fwd(a: Tensor, b: Tensor) -> Tuple[Tensor, Tensor]:
    """(out, stats): out = logsumexp_k(a + b); stats is the library's workspace."""
    B, M, K, N = _check(a, b)
    out = torch.empty(B, M, N, dtype=a.dtype, device=a.device)
    stats = torch.empty(_stats_size(B, M, K, N), dtype=_F32, device=a.device)
    _call("genbmm_logbmm_fwd" + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(stats), B, M, K, N)
    return out, stats


@logbmm_fwd.register_fake
def _(a, b):
    B, M, K, N = _dims(a, b)
    return a.new_empty(B, M, N), a.new_empty(_stats_size(B, M, K, N), dtype=_F32)


@torch.library.custom_op("genbmm_amd::logbmm_bwd", mutates_args=())
def logbmm_bwd(a: Tensor, b: Tensor, out: Tensor, g: Tensor, stats: Tensor) -> Tuple[Tensor, Tensor]:
    B, M, K, N = _check(a, b)
    g = g.to(a.dtype).contiguous()
    grad_a, grad_b = torch.empty_like(a), torch.empty_like(b)
    _call("genbmm_logbmm_bwd" + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(g), _lib.ptr(stats),
          _lib.ptr(grad_a), _lib.ptr(grad_b), B, M, K, N)
    return grad_a, grad_b


@logbmm_bwd.register_fake
def _(a, b, out, g, stats):
    return torch.empty_like(a), torch.empty_like(b)


@torch.library.custom_op("genbmm_amd::logbmm_bwdbwd", mutates_args=())
def logbmm_bwdbwd(a: Tensor, b: Tensor, out: Tensor, g: Tensor, u_a: Tensor,
                  u_b: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """Gradients of <u_a, grad_a> + <u_b, grad_b> with respect to (a, b, g)."""
    B, M, K, N = _check(a, b)
    g, u_a, u_b = g.to(a.dtype).contiguous(), u_a.to(a.dtype).contiguous(), u_b.to(a.dtype).contiguous()
    ga, gb, gg = torch.empty_like(a), torch.empty_like(b), torch.empty_like(g)
    ws = torch.empty(_lib.load().genbmm_logbmm_bwdbwd_ws_size(B, M, K, N), dtype=torch.float32, device=a.device)
    _call("genbmm_logbmm_bwdbwd_ws" + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(g), _lib.ptr(u_a),
          _lib.ptr(u_b), _lib.ptr(ga), _lib.ptr(gb), _lib.ptr(gg), _lib.ptr(ws), B, M, K, N)
    return ga, gb, gg


@logbmm_bwdbwd.register_fake
def _(a, b, out, g, u_a, u_b):
    return torch.empty_like(a), torch.empty_like(b), torch.empty_like(g)


def _logbmm_setup(ctx, inputs, output):
    a, b = inputs
    out, stats = output
    ctx.save_for_backward(a, b, out, stats)


def _logbmm_backward(ctx, g_out, g_stats):
    a, b, out, stats = ctx.saved_tensors
    return tuple(torch.ops.genbmm_amd.logbmm_bwd(a, b, out, g_out, stats))


def _logbmm_bwd_setup(ctx, inputs, output):
    a, b, out, g, _ = inputs
    ctx.save_for_backward(a, b, out, g)


def _logbmm_bwd_backward(ctx, u_a, u_b):
    a, b, out, g = ctx.saved_tensors
    u_a = torch.zeros_like(a) if u_a is None else u_a
    u_b = torch.zeros_like(b) if u_b is None else u_b
    ga, gb, gg = torch.ops.genbmm_amd.logbmm_bwdbwd(a, b, out, g, u_a, u_b)
    return ga, gb, None, gg, None


torch.library.register_autograd("genbmm_amd::logbmm_fwd", _logbmm_backward, setup_context=_logbmm_setup)
torch.library.register_autograd("genbmm_amd::logbmm_bwd", _logbmm_bwd_backward, setup_context=_logbmm_bwd_setup)


def logbmm(a: Tensor, b: Tensor) -> Tensor:
    return torch.ops.genbmm_amd.logbmm_fwd(a, b)[0]


# ------------------------------------------------------- max / sample / prod-max
@torch.library.custom_op("genbmm_amd::maxbmm_fwd", mutates_args=())
def maxbmm_fwd(a: Tensor, b: Tensor) -> Tuple[Tensor, Tensor]:
    B, M, K, N = _check(a, b)
    out = torch.empty(B, M, N, dtype=a.dtype, device=a.device)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=a.device)
    _call("genbmm_maxbmm_fwd" + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(idx), B, M, K, N)
    return out, idx


@maxbmm_fwd.register_fake
def _(a, b):
    B, M, K, N = _dims(a, b)
    return a.new_empty(B, M, N), a.new_empty(B, M, N, dtype=torch.int32)


@torch.library.custom_op("genbmm_amd::samplebmm_fwd", mutates_args=())
def samplebmm_fwd(a: Tensor, b: Tensor, seed: int, offset: int) -> Tuple[Tensor, Tensor]:
    B, M, K, N = _check(a, b)
    out = torch.empty(B, M, N, dtype=a.dtype, device=a.device)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=a.device)
    stats = torch.empty(int(_lib.load().genbmm_samplebmm_stats_size(int(B), int(M), int(K), int(N))),
                        dtype=_F32, device=a.device)
    _call("genbmm_samplebmm_fwd" + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(idx), _lib.ptr(stats),
          seed & 0xFFFFFFFFFFFFFFFF, offset & 0xFFFFFFFFFFFFFFFF, B, M, K, N)
    return out, idx


@samplebmm_fwd.register_fake
def _(a, b, seed, offset):
    B, M, K, N = _dims(a, b)
    return a.new_empty(B, M, N), a.new_empty(B, M, N, dtype=torch.int32)


@torch.library.custom_op("genbmm_amd::argmax_bwd", mutates_args=())
def argmax_bwd(idx: Tensor, g: Tensor, K: int) -> Tuple[Tensor, Tensor]:
    """One-hot(idx) * g summed over n (grad_a) and over m (grad_b)."""
    B, M, N = idx.shape
    g = g.contiguous()
    grad_a = torch.empty(B, M, K, dtype=g.dtype, device=g.device)
    grad_b = torch.empty(B, K, N, dtype=g.dtype, device=g.device)
    _call("genbmm_argmax_bwd" + _sfx(g), g, _lib.ptr(idx), _lib.ptr(g), _lib.ptr(grad_a), _lib.ptr(grad_b), B, M, K, N)
    return grad_a, grad_b


@argmax_bwd.register_fake
def _(idx, g, K):
    B, M, N = idx.shape
    return g.new_empty(B, M, K), g.new_empty(B, K, N)


def _argmax_setup(ctx, inputs, output):
    ctx.K = inputs[0].shape[2]
    ctx.save_for_backward(output[1])
    ctx.extra = len(inputs) - 2  # samplebmm_fwd also takes seed and offset


def _argmax_backward(ctx, g_out, g_idx):
    (idx,) = ctx.saved_tensors
    ga, gb = torch.ops.genbmm_amd.argmax_bwd(idx, g_out, ctx.K)
    return (ga, gb) + (None,) * ctx.extra


torch.library.register_autograd("genbmm_amd::maxbmm_fwd", _argmax_backward, setup_context=_argmax_setup)
torch.library.register_autograd("genbmm_amd::samplebmm_fwd", _argmax_backward, setup_context=_argmax_setup)


@torch.library.custom_op("genbmm_amd::prodmaxbmm_fwd", mutates_args=())
def prodmaxbmm_fwd(a: Tensor, b: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """(out, idx, factors): factors holds a[m, idx] and b[idx, n] per cell for the backward."""
    B, M, K, N = _check(a, b)
    out = torch.empty(B, M, N, dtype=a.dtype, device=a.device)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=a.device)
    factors = torch.empty(2, B, M, N, dtype=_F32, device=a.device)
    _call("genbmm_prodmaxbmm_fwd" + _sfx(a), a, _lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.ptr(idx), _lib.ptr(factors),
          B, M, K, N)
    return out, idx, factors


@prodmaxbmm_fwd.register_fake
def _(a, b):
    B, M, K, N = _dims(a, b)
    return a.new_empty(B, M, N), a.new_empty(B, M, N, dtype=torch.int32), a.new_empty(2, B, M, N, dtype=_F32)


@torch.library.custom_op("genbmm_amd::prodmax_bwd", mutates_args=())
def prodmax_bwd(idx: Tensor, factors: Tensor, g: Tensor, K: int) -> Tuple[Tensor, Tensor]:
    B, M, N = idx.shape
    g = g.contiguous()
    grad_a = torch.empty(B, M, K, dtype=g.dtype, device=g.device)
    grad_b = torch.empty(B, K, N, dtype=g.dtype, device=g.device)
    _call("genbmm_prodmax_bwd" + _sfx(g), g, _lib.ptr(None), _lib.ptr(None), _lib.ptr(idx), _lib.ptr(factors), _lib.ptr(g),
          _lib.ptr(grad_a), _lib.ptr(grad_b), B, M, K, N)
    return grad_a, grad_b


@prodmax_bwd.register_fake
def _(idx, factors, g, K):
    B, M, N = idx.shape
    return g.new_empty(B, M, K), g.new_empty(B, K, N)


def _prodmax_setup(ctx, inputs, output):
    ctx.K = inputs[0].shape[2]
    ctx.save_for_backward(output[1], output[2])


def _prodmax_backward(ctx, g_out, g_idx, g_fac):
    idx, factors = ctx.saved_tensors
    return tuple(torch.ops.genbmm_amd.prodmax_bwd(idx, factors, g_out, ctx.K))


torch.library.register_autograd("genbmm_amd::prodmaxbmm_fwd", _prodmax_backward, setup_context=_prodmax_setup)


def maxbmm(a: Tensor, b: Tensor) -> Tensor:
    return torch.ops.genbmm_amd.maxbmm_fwd(a, b)[0]


def prodmaxbmm(a: Tensor, b: Tensor) -> Tensor:
    return torch.ops.genbmm_amd.prodmaxbmm_fwd(a, b)[0]


def samplebmm(a: Tensor, b: Tensor, seed: int, offset: int = 0) -> Tensor:
    """The Philox stream (seed, offset) is an explicit argument: a traced graph must not
    read the global generator."""
    return torch.ops.genbmm_amd.samplebmm_fwd(a, b, seed, offset)[0]


# ----------------------------------------------------------------------- banded
# The three banded products of genbmm_amd.sparse (reference sparse.py:404-637) as
# operators on the band tensors themselves: a (B, n, a_lu + a_ld + 1), b likewise.
# mode: 0 log, 1 max, 3 (+,*) - the library's GENBMM_BAND_* values.
_BAND_LOG, _BAND_MAX, _BAND_MUL = 0, 1, 3


def _band_dims(a: Tensor, b: Tensor, a_lu: int, a_ld: int, b_lu: int, b_ld: int):
    if a.dtype != _F32 or b.dtype != _F32:
        raise RuntimeError("genbmm_amd.ops: float32 tensors only (use BandedMatrix for others)")
    if a.dim() != 3 or b.dim() != 3 or a.shape[:2] != b.shape[:2]:
        raise RuntimeError("band tensors must be (batch, n, width) with equal batch and n")
    if a.shape[2] != a_lu + a_ld + 1 or b.shape[2] != b_lu + b_ld + 1:
        raise RuntimeError("band widths do not match lu + ld + 1")
    return a.shape[0], a.shape[1], a.shape[2] + b.shape[2] - 1


def _band_ws_size(a_lu, a_ld, b_lu, b_ld, B, n):
    return int(_lib.load().genbmm_banded_workspace_size(int(a_lu), int(a_ld), int(b_lu), int(b_ld), int(B), int(n)))


@torch.library.custom_op("genbmm_amd::banded_fwd", mutates_args=())
def banded_fwd(a: Tensor, b: Tensor, a_lu: int, a_ld: int, b_lu: int, b_ld: int, mode: int) -> Tuple[Tensor, Tensor]:
    """(out, aux): the product's band tensor (lu = a_lu + b_ld, ld = a_ld + b_lu) and what the
    backward needs beside the operands - the arg-max (int32) for max, the library's
    workspace for log, nothing (an empty tensor) for (+,*)."""
    B, n, wo = _band_dims(a, b, a_lu, a_ld, b_lu, b_ld)
    a, b = a.contiguous(), b.contiguous()
    out = torch.empty(B, n, wo, dtype=_F32, device=a.device)
    if mode == _BAND_MAX:
        aux = torch.empty(B, n, wo, dtype=torch.int32, device=a.device)
        idx, ws = aux, None
    elif mode == _BAND_LOG:
        aux = torch.empty(_band_ws_size(a_lu, a_ld, b_lu, b_ld, B, n), dtype=_F32, device=a.device)
        idx, ws = None, aux
    else:
        aux = torch.empty(0, dtype=_F32, device=a.device)
        idx, ws = None, None
    _call("genbmm_banded_fwd", a, _lib.ptr(a), a_lu, a_ld, _lib.ptr(b), b_lu, b_ld, _lib.ptr(out), _lib.ptr(idx),
          _lib.ptr(ws), B, n, mode)
    return out, aux


@banded_fwd.register_fake
def _(a, b, a_lu, a_ld, b_lu, b_ld, mode):
    B, n, wo = a.shape[0], a.shape[1], a.shape[2] + b.shape[2] - 1
    if mode == _BAND_MAX:
        aux = a.new_empty((B, n, wo), dtype=torch.int32)
    elif mode == _BAND_LOG:
        aux = a.new_empty(_band_ws_size(a_lu, a_ld, b_lu, b_ld, B, n))
    else:
        aux = a.new_empty(0)
    return a.new_empty(B, n, wo), aux


@torch.library.custom_op("genbmm_amd::banded_bwd", mutates_args=())
def banded_bwd(a: Tensor, b: Tensor, out: Tensor, aux: Tensor, g: Tensor, a_lu: int, a_ld: int, b_lu: int,
               b_ld: int, mode: int) -> Tuple[Tensor, Tensor]:
    """(grad_a, grad_b).  For the log product the library keeps g / sum per output cell
    beside the workspace: in a buffer of this call's own, so that `aux` is only read."""
    B, n, wo = _band_dims(a, b, a_lu, a_ld, b_lu, b_ld)
    a, b, g = a.contiguous(), b.contiguous(), g.contiguous()
    grad_a, grad_b = torch.empty_like(a), torch.empty_like(b)
    idx = aux if mode == _BAND_MAX else None
    ws = aux if mode == _BAND_LOG else None
    o = out if mode == _BAND_LOG else None
    scratch = None
    if mode == _BAND_LOG:
        need = int(_lib.load().genbmm_banded_scratch_size(int(a_lu), int(a_ld), int(b_lu), int(b_ld), int(B), int(n)))
        scratch = torch.empty(need, dtype=_F32, device=a.device) if need else None
    _call("genbmm_banded_bwd_scratch", a, _lib.ptr(a), a_lu, a_ld, _lib.ptr(b), b_lu, b_ld, _lib.ptr(o),
          _lib.ptr(idx), _lib.ptr(ws), _lib.ptr(scratch), _lib.ptr(g), _lib.ptr(grad_a), _lib.ptr(grad_b), B, n, mode)
    return grad_a, grad_b


@banded_bwd.register_fake
def _(a, b, out, aux, g, a_lu, a_ld, b_lu, b_ld, mode):
    return torch.empty_like(a), torch.empty_like(b)


@torch.library.custom_op("genbmm_amd::banded_bwdbwd", mutates_args=())
def banded_bwdbwd(a: Tensor, b: Tensor, out: Tensor, g: Tensor, u_a: Tensor, u_b: Tensor, a_lu: int, a_ld: int,
                  b_lu: int, b_ld: int) -> Tuple[Tensor, Tensor, Tensor]:
    """Log product: gradients of <u_a, grad_a> + <u_b, grad_b> with respect to (a, b, g)."""
    B, n, _ = _band_dims(a, b, a_lu, a_ld, b_lu, b_ld)
    a, b, g, u_a, u_b = a.contiguous(), b.contiguous(), g.contiguous(), u_a.contiguous(), u_b.contiguous()
    ga, gb, gg = torch.empty_like(a), torch.empty_like(b), torch.empty_like(g)
    _call("genbmm_banded_bwdbwd", a, _lib.ptr(a), a_lu, a_ld, _lib.ptr(b), b_lu, b_ld, _lib.ptr(out), _lib.ptr(g),
          _lib.ptr(u_a), _lib.ptr(u_b), _lib.ptr(ga), _lib.ptr(gb), _lib.ptr(gg), B, n)
    return ga, gb, gg


@banded_bwdbwd.register_fake
def _(a, b, out, g, u_a, u_b, a_lu, a_ld, b_lu, b_ld):
    return torch.empty_like(a), torch.empty_like(b), torch.empty_like(g)


def _banded_setup(ctx, inputs, output):
    a, b, a_lu, a_ld, b_lu, b_ld, mode = inputs
    out, aux = output
    ctx.save_for_backward(a, b, out, aux)
    ctx.band = (a_lu, a_ld, b_lu, b_ld, mode)


def _banded_backward(ctx, g_out, g_aux):
    a, b, out, aux = ctx.saved_tensors
    ga, gb = torch.ops.genbmm_amd.banded_bwd(a, b, out, aux, g_out, *ctx.band)
    return ga, gb, None, None, None, None, None


def _banded_bwd_setup(ctx, inputs, output):
    a, b, out, _, g, a_lu, a_ld, b_lu, b_ld, mode = inputs
    ctx.save_for_backward(a, b, out, g)
    ctx.band = (a_lu, a_ld, b_lu, b_ld, mode)


def _banded_bwd_backward(ctx, u_a, u_b):
    a, b, out, g = ctx.saved_tensors
    a_lu, a_ld, b_lu, b_ld, mode = ctx.band
    if mode != _BAND_LOG:  # as in the reference: only the log product has second-order terms
        raise RuntimeError("genbmm_amd.ops: only the banded log product is twice differentiable")
    u_a = torch.zeros_like(a) if u_a is None else u_a
    u_b = torch.zeros_like(b) if u_b is None else u_b
    ga, gb, gg = torch.ops.genbmm_amd.banded_bwdbwd(a, b, out, g, u_a, u_b, a_lu, a_ld, b_lu, b_ld)
    return ga, gb, None, None, gg, None, None, None, None, None


torch.library.register_autograd("genbmm_amd::banded_fwd", _banded_backward, setup_context=_banded_setup)
torch.library.register_autograd("genbmm_amd::banded_bwd", _banded_bwd_backward, setup_context=_banded_bwd_setup)


def banded_multiply(a: Tensor, a_lu: int, a_ld: int, b: Tensor, b_lu: int, b_ld: int) -> Tensor:
    """Band tensor of the (+,*) product; its band is (a_lu + b_ld, a_ld + b_lu)."""
    return torch.ops.genbmm_amd.banded_fwd(a, b, a_lu, a_ld, b_lu, b_ld, _BAND_MUL)[0]


def banded_multiply_log(a: Tensor, a_lu: int, a_ld: int, b: Tensor, b_lu: int, b_ld: int) -> Tensor:
    return torch.ops.genbmm_amd.banded_fwd(a, b, a_lu, a_ld, b_lu, b_ld, _BAND_LOG)[0]


def banded_multiply_max(a: Tensor, a_lu: int, a_ld: int, b: Tensor, b_lu: int, b_ld: int) -> Tensor:
    return torch.ops.genbmm_amd.banded_fwd(a, b, a_lu, a_ld, b_lu, b_ld, _BAND_MAX)[0]
