"""Build step: compile the HIP sources into libgenbmm_gfx950.so (in-tree).

    python -m genbmm_amd.build

This takes the place of the reference's setup.py (setup.py:1-27, a
torch CUDAExtension named `_genbmm`): there is no pybind11 / torch extension
here, only a plain shared library with a C ABI (include/genbmm_gfx950.h) that
genbmm_amd/_lib.py loads with ctypes.  hipcc cross-compiles for gfx950 without
a GPU being present.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBNAME = "libgenbmm_gfx950.so"
SOURCES = ["logbmm.hip", "logbmm_bb.hip", "dense_fwd.hip", "dense_bwd.hip", "banded.hip", "band_struct.hip", "f64.hip"]
# Sources that are compiled once per element type of the caller's tensors: float (entry points
# genbmm_*), IEEE binary16 (genbmm_*_f16) and bfloat16 (genbmm_*_bf16); see csrc/common.h.
_ELEMENTS = (("", 0), ("_f16", 1), ("_bf16", 2))
PER_ELEMENT = {"logbmm.hip": _ELEMENTS, "logbmm_bb.hip": _ELEMENTS, "dense_fwd.hip": _ELEMENTS, "dense_bwd.hip": _ELEMENTS,
               "banded.hip": _ELEMENTS}

# -packed-fp32-ops is switched OFF: v_pk_{add,mul,fma}_f32 are not used by any
# kernel here, and the compiler must not form them on its own either.
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    # multiply-add fusion only where the source spells fmaf(): kernels whose results
    # must be bit-exact round each product before adding it
    "-ffp-contract=on",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fno-gpu-rdc",
    "-Wno-unused-command-line-argument",
]


# Per-source additions.  The banded kernels keep their 16 x 16 accumulators in ordinary vector
# registers: a tile's four values are read by vector instructions right after its last matrix
# instruction, and copies to and from the accumulation registers around every step cost
# more than the registers they free.
EXTRA_FLAGS = {"banded.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def lib_path():
    return os.path.join(LIBDIR, LIBNAME)


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; it is needed to build " + LIBNAME)
    return exe


def build(verbose=True):
    """Compile every source for gfx950 and link the shared library. Always recompiles."""
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    cc = hipcc()
    procs = []
    for src in SOURCES:
        for suffix, elem in PER_ELEMENT.get(src, (("", 0),)):
            obj = os.path.join(objdir, src.replace(".hip", suffix + ".o"))
            cmd = ([cc] + HIPCC_FLAGS + EXTRA_FLAGS.get(src, []) + ["-DGENBMM_ELEM=%d" % elem, "-c",
                   os.path.join(CSRC, src), "-o", obj])
            if verbose:
                print(" ".join(cmd), flush=True)
            procs.append((src + suffix, obj,
                          subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    objs = []
    for src, obj, proc in procs:
        out = proc.communicate()[0].decode()
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        objs.append(obj)
    tmp = lib_path() + ".tmp"
    cmd = [cc, "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-rdc"] + objs + ["-o", tmp]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    os.replace(tmp, lib_path())
    return lib_path()


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
