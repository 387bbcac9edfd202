"""ctypes binding of libgenbmm_gfx950.so and the argument checks in front of it.

Takes the place of the reference's pybind11 module `_genbmm`
(matmul_cuda.cpp:165-172).  The reference checks `is_cuda` and `is_contiguous`
and raises RuntimeError (matmul_cuda.cpp:65-67); the checks here raise
RuntimeError for the same conditions and additionally for dtype / shape
disagreement, which the reference leaves to undefined behaviour.

There is no CPU path: calling any op without the library, or with CPU tensors,
raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libgenbmm_gfx950.so")

_c_float_p = ctypes.c_void_p
_c_int_p = ctypes.c_void_p
_i = ctypes.c_int
_u64 = ctypes.c_uint64
_vp = ctypes.c_void_p

_DENSE_DIMS = [_i, _i, _i, _i, _vp]  # B, M, K, N, stream
_BAND = [_c_float_p, _i, _i, _c_float_p, _i, _i]  # a, a_lu, a_ld, b, b_lu, b_ld

# name -> argtypes (every function returns int unless noted); mirrors
# include/genbmm_gfx950.h
SIGNATURES = {
    "genbmm_logbmm_fwd": [_c_float_p] * 4 + _DENSE_DIMS,
    "genbmm_logbmm_bwd": [_c_float_p] * 7 + _DENSE_DIMS,
    "genbmm_logbmm_fwd_static": [_c_float_p] * 3 + _DENSE_DIMS,
    "genbmm_logbmm_fwd_path": [_c_float_p] * 4 + [_i, _i, _i, _i, _i, _vp],  # ..., B, M, K, N, path, stream
    "genbmm_logbmm_bwd_path": [_c_float_p] * 7 + [_i, _i, _i, _i, _i, _vp],
    "genbmm_logbmm_bwdbwd": [_c_float_p] * 9 + _DENSE_DIMS,
    "genbmm_logbmm_bwdbwd_ws": [_c_float_p] * 10 + _DENSE_DIMS,
    "genbmm_maxbmm_fwd": [_c_float_p] * 3 + [_c_int_p] + _DENSE_DIMS,
    "genbmm_prodmaxbmm_fwd": [_c_float_p] * 3 + [_c_int_p, _c_float_p] + _DENSE_DIMS,
    "genbmm_samplebmm_fwd": [_c_float_p] * 3 + [_c_int_p, _c_float_p, _u64, _u64] + _DENSE_DIMS,
    "genbmm_argmax_bwd": [_c_int_p] + [_c_float_p] * 3 + _DENSE_DIMS,
    "genbmm_prodmax_bwd": [_c_float_p] * 2 + [_c_int_p] + [_c_float_p] * 4 + _DENSE_DIMS,
    "genbmm_banded_fwd": _BAND + [_c_float_p, _c_int_p, _c_float_p, _i, _i, _i, _vp],
    "genbmm_banded_sample_fwd": _BAND + [_c_float_p, _c_int_p, _c_float_p, _u64, _u64, _i, _i, _vp],
    "genbmm_banded_bwd": _BAND + [_c_float_p, _c_int_p] + [_c_float_p] * 4 + [_i, _i, _i, _vp],
    "genbmm_banded_bwd_scratch": _BAND + [_c_float_p, _c_int_p] + [_c_float_p] * 5 + [_i, _i, _i, _vp],
    "genbmm_banded_bwdbwd": _BAND + [_c_float_p] * 7 + [_i, _i, _vp],
    "genbmm_logbmm_fwd_f64": [_c_float_p] * 3 + _DENSE_DIMS,
    "genbmm_logbmm_bwd_f64": [_c_float_p] * 6 + _DENSE_DIMS,
    "genbmm_logbmm_bwdbwd_f64": [_c_float_p] * 9 + _DENSE_DIMS,
    "genbmm_maxbmm_fwd_f64": [_c_float_p] * 3 + [_c_int_p] + _DENSE_DIMS,
    "genbmm_prodmaxbmm_fwd_f64": [_c_float_p] * 3 + [_c_int_p] + _DENSE_DIMS,
    "genbmm_samplebmm_fwd_f64": [_c_float_p] * 3 + [_c_int_p, _u64, _u64] + _DENSE_DIMS,
    "genbmm_argmax_bwd_f64": [_c_int_p] + [_c_float_p] * 3 + _DENSE_DIMS,
    "genbmm_prodmax_bwd_f64": [_c_float_p] * 2 + [_c_int_p] + [_c_float_p] * 3 + _DENSE_DIMS,
    "genbmm_banded_fwd_f64": _BAND + [_c_float_p, _c_int_p, _i, _i, _i, _vp],
    "genbmm_banded_sample_fwd_f64": _BAND + [_c_float_p, _c_int_p, _u64, _u64, _i, _i, _vp],
    "genbmm_banded_bwd_f64": _BAND + [_c_float_p, _c_int_p] + [_c_float_p] * 3 + [_i, _i, _i, _vp],
    "genbmm_banded_bwdbwd_f64": _BAND + [_c_float_p] * 7 + [_i, _i, _vp],
    "genbmm_band_shift": [_c_float_p, _c_float_p] + [_i] * 6 + [ctypes.c_float, _vp],
    "genbmm_band_op": _BAND + [_c_float_p, _i, _i, _i, ctypes.c_float, _vp],
    "genbmm_band_transpose": [_c_float_p, _c_float_p, _i, _i, _i, _i, _vp],
    "genbmm_band_to_dense": [_c_float_p, _c_float_p, _i, _i, _i, _i, ctypes.c_float, _vp],
    "genbmm_band_from_dense": [_c_float_p, _c_float_p, _i, _i, _i, _i, _i, _vp],
}
# Entry points that also exist for float16 (`*_f16`) and bfloat16 (`*_bf16`) tensors: the same
# arguments, the caller's tensors in that type, every workspace still float32.
HALF_VARIANTS = ("genbmm_logbmm_fwd", "genbmm_logbmm_bwd", "genbmm_logbmm_fwd_path", "genbmm_logbmm_bwd_path",
                 "genbmm_maxbmm_fwd", "genbmm_prodmaxbmm_fwd", "genbmm_samplebmm_fwd", "genbmm_argmax_bwd",
                 "genbmm_prodmax_bwd", "genbmm_logbmm_bwdbwd_ws", "genbmm_banded_fwd", "genbmm_banded_sample_fwd", "genbmm_banded_bwd",
                 "genbmm_banded_bwd_scratch")
for _name in HALF_VARIANTS:
    for _suffix in ("_f16", "_bf16"):
        SIGNATURES[_name + _suffix] = SIGNATURES[_name]
for _suffix in ("_f16", "_bf16"):  # one more buffer than the float function: t_scratch (B * n * Wo floats)
    SIGNATURES["genbmm_banded_bwdbwd" + _suffix] = _BAND + [_c_float_p] * 8 + [_i, _i, _vp]
HALF_SUFFIX = {torch.float16: "_f16", torch.bfloat16: "_bf16"}
STRING_FUNCS = {"genbmm_version": [], "genbmm_error_string": [_i]}
INT_FUNCS = {"genbmm_logbmm_fwd_pieces": [_i, _i, _i, _i], "genbmm_maxbmm_fwd_pieces": [_i, _i, _i, _i],
             "genbmm_banded_on_matrix_cores": [_i, _i, _i, _i, _i, _i]}
SIZE_FUNCS = {"genbmm_logbmm_stats_size": [_i, _i, _i, _i],
              "genbmm_logbmm_bwdbwd_ws_size": [_i, _i, _i, _i],
              "genbmm_logbmm_stats_size_path": [_i, _i, _i, _i, _i],
              "genbmm_samplebmm_stats_size": [_i, _i, _i, _i],
              "genbmm_logbmm_static_limit": [],
              "genbmm_banded_workspace_size": [_i, _i, _i, _i, _i, _i],
              "genbmm_banded_scratch_size": [_i, _i, _i, _i, _i, _i]}

_lib = None


def load():
    """Load the shared library (once). Raises RuntimeError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "genbmm_amd: %s is missing; build it with `python -m genbmm_amd.build` "
            "(there is no CPU or PyTorch fallback)" % LIB_PATH
        )
    # torch is imported above, so its HIP runtime (libamdhip64.so.7) is already
    # mapped and the library binds to that copy rather than loading a second one.
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    for name, argtypes in STRING_FUNCS.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_char_p
    for name, argtypes in INT_FUNCS.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    for name, argtypes in SIZE_FUNCS.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_size_t
    _lib = lib
    return lib


def version():
    return load().genbmm_version().decode()


def check(code, what):
    if code != 0:
        msg = load().genbmm_error_string(code).decode()
        raise RuntimeError("genbmm_amd: %s failed (%d): %s" % (what, code, msg))


def stream_of(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def require(t, name, dtype=torch.float32, ndim=3, device=None):
    """Device / layout / dtype checks (reference CHECK_INPUT, matmul_cuda.cpp:65-67)."""
    if not isinstance(t, torch.Tensor):
        raise RuntimeError("%s must be a tensor" % name)
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    if t.dtype != dtype:
        raise RuntimeError("%s must be %s, got %s" % (name, dtype, t.dtype))
    if ndim is not None and t.dim() != ndim:
        raise RuntimeError("%s must have %d dimensions, got %d" % (name, ndim, t.dim()))
    if device is not None and t.device != device:
        raise RuntimeError("%s is on %s, expected %s" % (name, t.device, device))
    return t


def dense_dims(a, b):
    """(B, M, K, N) of a (B,M,K) x (B,K,N) product, with agreement checks; a's element
    type (float32, float64, float16 or bfloat16) is the one both must have."""
    dtype = torch.float32
    if isinstance(a, torch.Tensor) and (a.dtype == torch.float64 or a.dtype in HALF_SUFFIX):
        dtype = a.dtype
    require(a, "a", dtype=dtype)
    require(b, "b", dtype=dtype, device=a.device)
    B, M, K = a.shape
    if b.shape[0] != B or b.shape[1] != K:
        raise RuntimeError(
            "shape mismatch: a is %s, b is %s" % (tuple(a.shape), tuple(b.shape))
        )
    return B, M, K, b.shape[2]


class device_of:
    """Make the tensors' device current around a library call (the reference has no guard)."""

    def __init__(self, t):
        self.guard = torch.cuda.device(t.device)

    def __enter__(self):
        self.guard.__enter__()

    def __exit__(self, *exc):
        return self.guard.__exit__(*exc)
