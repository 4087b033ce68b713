"""The library's host encoder (the product) against the oracle, bit for bit.  No GPU."""
import numpy as np
import pytest
import torch

import ternainfer_amd as T
from oracle import terna_oracle as O
from tests._util import make_row_skewed, make_ternary


def _same(a, b):
    for x, y in zip(a, b):
        x = x.numpy()
        assert x.dtype == y.dtype and x.shape == y.shape and (x == y).all()


@pytest.mark.parametrize("shape,p0,seed", [((64, 64), 0.45, 1), ((128, 192), 0.40, 2), ((256, 320), 0.2, 3),
                                           ((64, 128), 1.0, 4), ((64, 128), 0.0, 5)])
def test_compress_weight_matches_oracle(coracle, shape, p0, seed):
    w = make_ternary(*shape, p0, seed)
    got = T.compress_weight(torch.from_numpy(w))
    _same(got, coracle.encode(w))
    _same(got, O.encode(w))
    vals, off, med, bm = got
    assert (vals.dtype, off.dtype, med.dtype, bm.dtype) == (torch.uint32, torch.int32, torch.uint16, torch.uint64)


def test_compress_weight_row_skewed_round_trip(coracle):
    w = make_row_skewed(256, 192, 9)
    vals, off, med, bm = [t.numpy() for t in T.compress_weight(torch.from_numpy(w))]
    assert (coracle.decode(vals, off, med, bm, 256, 192) == w).all()


def test_reorder_weight_matches_oracle(coracle):
    w = make_ternary(64, 96 + 32, 0.3, 6)
    assert (T.reorder_weight(torch.from_numpy(w)).numpy() == coracle.reorder(w)).all()


def test_golden_fixture(coracle):
    """tests/golden/format_128x192.npz: W and its encoding as written by the oracle
    (tests/golden/make_golden.py); the library's encoder and both oracle decoders must agree."""
    import os
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "format_128x192.npz"))
    w = g["w"]
    got = T.compress_weight(torch.from_numpy(w))
    _same(got, (g["compressed_val"], g["tile_offsets_global"], g["tile_offsets_median"], g["bitmap"]))
    assert (coracle.decode(g["compressed_val"], g["tile_offsets_global"], g["tile_offsets_median"], g["bitmap"],
                           *w.shape) == w).all()


def test_rejects_non_ternary_and_bad_shape():
    with pytest.raises(ValueError):
        T.compress_weight(torch.full((64, 64), 2, dtype=torch.int8))
    with pytest.raises(ValueError):
        T.compress_weight(torch.zeros((64, 96), dtype=torch.int8))


def test_quant_weight_and_scale_packing():
    g = torch.Generator().manual_seed(3)
    w = torch.randn(64, 64, generator=g) * 0.02
    t, sc = T.quant_weight_int8(w)
    t_o, sc_o = O.quant_weight_int8(w.numpy())
    assert (t.numpy() == t_o).all() and set(np.unique(t.numpy())) <= {-1, 0, 1}
    assert abs(float(sc) - float(sc_o)) <= 2 ** -8 * float(sc_o)
    ws = T.pack_weight_scale([sc, sc])
    assert ws.dtype == torch.bfloat16 and ws.shape == (4,) and int((ws != 0).sum()) == 2
