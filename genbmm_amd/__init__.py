"""genbmm for AMD MI355X (gfx950): generalized-semiring batched matmul and banded
matrices for PyTorch-ROCm, as hand-written HIP kernels behind a C ABI.

Exports the same six names as the reference package (genbmm/__init__.py:1-4).
`install_as_genbmm()` additionally registers this package under the name
`genbmm`, so that code written against the reference (`import genbmm`) runs
unchanged.
"""
import sys

from .genmul import logbmm, samplebmm, maxbmm, prodmaxbmm
from .sparse import BandedMatrix, banddiag

__all__ = ["logbmm", "samplebmm", "maxbmm", "prodmaxbmm", "BandedMatrix", "banddiag"]
__version__ = "0.1"


def install_as_genbmm():
    """Make `import genbmm` resolve to this package (no-op if already done)."""
    me = sys.modules[__name__]
    other = sys.modules.get("genbmm")
    if other is not None and other is not me:
        raise RuntimeError("a different `genbmm` module is already imported")
    sys.modules["genbmm"] = me
    sys.modules["genbmm.genmul"] = sys.modules[__name__ + ".genmul"]
    sys.modules["genbmm.sparse"] = sys.modules[__name__ + ".sparse"]
    return me
