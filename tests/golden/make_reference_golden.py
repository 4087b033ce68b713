"""Writes tests/golden/reference_format_*.npz by running the REFERENCE's own Python encoder
(/root/reference/convert/convert_utils.py: reorder_weight + compress_weight) on small seeded matrices.

Run in the build container only, from the repository root:  python tests/golden/make_reference_golden.py
The reference tree does not exist anywhere else; the fixtures it leaves are plain data (inputs, the four output arrays,
their torch dtypes and shapes) and are what the tests read.

What this pins that nothing else does: the serialised form of a converted tensor as the reference writes it -- element
types (uint32 / int32 / uint16 / uint64), one-dimensional shapes, and the zero-length TileOffsets_median of a
matrix without any nonzero (convert_utils.py:226) -- and, once more and by the reference's own code instead of
a restatement, the bit-level content of the four arrays.  tests/test_oracle_format.py and tests/test_host_encoder.py
compare the oracle's encoders and the library's host encoder with these files.
"""
import importlib.util
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = "/root/reference/convert/convert_utils.py"

from tests._util import make_row_skewed, make_ternary  # noqa: E402


def as_numpy(t: torch.Tensor) -> np.ndarray:
    """Same bytes, numpy's unsigned types where torch has them only as storage."""
    names = {torch.uint16: np.uint16, torch.uint32: np.uint32, torch.uint64: np.uint64}
    if t.dtype in names:
        signed = {torch.uint16: torch.int16, torch.uint32: torch.int32, torch.uint64: torch.int64}[t.dtype]
        return t.view(signed).numpy().view(names[t.dtype]).copy()
    return t.numpy().copy()


def main():
    spec = importlib.util.spec_from_file_location("reference_convert_utils", REFERENCE)
    ref = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ref)
    cases = {
        "64x128_p40": make_ternary(64, 128, 0.40, 20260011),
        "128x192_p45": make_ternary(128, 192, 0.45, 20260012),
        "128x128_skewed": make_row_skewed(128, 128, 20260013),
        "64x64_dense": make_ternary(64, 64, 0.0, 20260014),
        "64x128_empty": np.zeros((64, 128), np.int8),
    }
    for name, w in cases.items():
        reordered = ref.reorder_weight(torch.from_numpy(w))
        vals, off, med, bm = ref.compress_weight(torch.from_numpy(w))
        np.savez_compressed(
            os.path.join(HERE, f"reference_format_{name}.npz"), w=w, reordered=reordered.numpy(),
            compressed_val=as_numpy(vals), tile_offsets_global=as_numpy(off), tile_offsets_median=as_numpy(med),
            bitmap=as_numpy(bm),
            torch_dtypes=np.array([str(t.dtype) for t in (vals, off, med, bm)]),
            torch_shapes=np.array([str(tuple(t.shape)) for t in (vals, off, med, bm)]))
        print(name, [str(t.dtype) for t in (vals, off, med, bm)], [tuple(t.shape) for t in (vals, off, med, bm)])


if __name__ == "__main__":
    main()
