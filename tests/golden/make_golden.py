"""Writes tests/golden/*.npz.  Run from the repository root:  python tests/golden/make_golden.py

Provenance: the reference stores no golden vectors for this path and its Python encoder is
read, not run (its arithmetic is pinned by closed forms and by the replay of the reference
kernel's consumer in tests/test_oracle_format.py).  These fixtures are therefore written by
the oracle, once that pinning is green.  They are DRIFT GUARDS ONLY: they freeze the byte-level
format and two small linear layers against later changes in the oracle or the library, and
pin nothing about the oracle itself -- a mistake the oracle had when they were written would
be frozen with them.  What pins the oracle are the hand-worked and closed-form checks in
tests/test_oracle_format.py and tests/test_oracle_linear.py.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import terna_oracle as O  # noqa: E402
from tests._util import make_bf16_activations, make_int8_activations, make_ternary  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    c = O.COracle()
    w = make_ternary(128, 192, 0.40, 20260001)
    vals, off, med, bm = c.encode(w)
    assert all((a == b).all() for a, b in zip((vals, off, med, bm), O.encode(w)))
    np.savez_compressed(os.path.join(HERE, "format_128x192.npz"), w=w, compressed_val=vals,
                        tile_offsets_global=off, tile_offsets_median=med, bitmap=bm)

    # one small linear layer in both families: inputs and oracle outputs
    xq, s = make_int8_activations(8, 192, 20260002)
    ws = O.f32_to_bf16_bits(np.array([0.75, 1.5, 0, 0], dtype=np.float32))
    out_dec = c.spmm_i8(xq, w, s, ws, 2, 0)
    out_pre = c.spmm_i8(xq, w, s, ws, 2, 1)
    xb = make_bf16_activations(8, 192, 20260003)
    scale = np.array([1.25], dtype=np.float32)
    ref = c.spmm_bf16(xb, w, scale, 1)
    np.savez_compressed(os.path.join(HERE, "linear_8x128x192.npz"), x_q=xq, s=s, ws=ws, ws_num=2,
                        out_i8_decode=out_dec, out_i8_prefill=out_pre, x_bf16=xb, scale=scale, ref_fp64=ref)
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


if __name__ == "__main__":
    main()
