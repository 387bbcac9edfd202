"""Writes tests/golden/band_struct.npz: input / output vectors of the reference's
structural BandedMatrix methods that the reference itself never tests (band_shift,
band_pad, band_unshift, col_shift, col_unshift, _expand, op, transpose, to_dense;
genbmm/sparse.py:81-218) plus its CPU Python-loop products (multiply_simple,
multiply_log_simple, multiply_max_simple, multiply_back_simple; sparse.py:268-401).

Run in the build container only (it imports the reference's pure-Python module from
/root/reference on the CPU; no compiled extension is involved):

    python tests/golden/make_band_struct_fixtures.py

The fixture holds data only; tests/test_host.py and tests/test_oracle.py read it with
numpy.load(allow_pickle=False).
"""
import os
import sys

import numpy as np
import torch

REF = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    sys.path.insert(0, REF)
    from genbmm.sparse import BandedMatrix, banddiag  # noqa: E402  (the reference's own code)

    g = torch.Generator().manual_seed(20240607)
    out = {}
    cases = [(2, 7, 2, 3, 0.0), (1, 5, 0, 2, -1e9), (3, 9, 3, 1, 0.0), (2, 6, 1, 1, -1e9)]
    out["n_cases"] = np.array(len(cases))
    for c, (B, n, lu, ld, fill) in enumerate(cases):
        dense = torch.randn(B, n, n, generator=g)
        band = banddiag(dense, lu, ld, fill)[0].clone()
        bm = BandedMatrix(band, lu, ld, fill)
        other_lu, other_ld = ld, lu + 1
        oband = banddiag(torch.randn(B, n, n, generator=g), other_lu, other_ld, fill)[0].clone()
        om = BandedMatrix(oband, other_lu, other_ld, fill)
        p = "c%d_" % c
        out[p + "meta"] = np.array([B, n, lu, ld, other_lu, other_ld], dtype=np.int64)
        out[p + "fill"] = np.array(fill, dtype=np.float64)
        out[p + "band"] = band.numpy()
        out[p + "oband"] = oband.numpy()

        def put(name, m):
            out[p + name] = m.data.contiguous().numpy()
            out[p + name + "_luld"] = np.array([m.lu, m.ld], dtype=np.int64)

        put("band_shift_p1", bm.band_shift(1))
        put("band_shift_m2", bm.band_shift(-2))
        put("band_pad_2", bm.band_pad(2))
        put("band_unshift", bm.band_unshift())
        put("col_shift_p1", bm.col_shift(1))
        put("col_shift_m2", bm.col_shift(-2))
        put("col_unshift", bm.col_unshift())
        put("expand", bm._expand(lu + 2, ld + 1))
        put("op_add", bm.op(om, lambda x, y: x + y, zero=0))
        put("op_max", bm.op(om, torch.max, zero=-1e9))
        put("transpose", bm.transpose())
        out[p + "to_dense"] = bm.to_dense().numpy()
        # the reference's CPU products (triple Python loops)
        zb = BandedMatrix(banddiag(dense, lu, ld, 0)[0].clone(), lu, ld, 0)
        zo = BandedMatrix(oband.clone().masked_fill(oband <= -1e8, 0.0), other_lu, other_ld, 0)
        out[p + "zband"] = zb.data.numpy()
        out[p + "zoband"] = zo.data.numpy()
        put("multiply_simple", zb.multiply_simple(zo))
        put("multiply_log_simple", zb.multiply_log_simple(zo))
        put("multiply_max_simple", zb.multiply_max_simple(zo))
        r = zb.multiply_simple(zo)
        gout = torch.randn(r.data.shape, generator=g)
        out[p + "grad_out"] = gout.numpy()
        put("multiply_back_simple", zb.multiply_back_simple(zo, BandedMatrix(gout, r.lu, r.ld, 0)))
    np.savez_compressed(os.path.join(HERE, "band_struct.npz"), **out)
    print("wrote", os.path.join(HERE, "band_struct.npz"), len(out), "arrays")


if __name__ == "__main__":
    main()
