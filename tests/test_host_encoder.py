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


REFERENCE_FIXTURES = ["64x128_p40", "128x192_p45", "128x128_skewed", "64x64_dense", "64x128_empty"]


@pytest.mark.parametrize("name", REFERENCE_FIXTURES)
def test_reference_written_fixtures(coracle, name):
    """tests/golden/reference_format_*.npz were written by the REFERENCE's own encoder (convert/convert_utils.py:9-228,
    run once in the build container by tests/golden/make_reference_golden.py).  Both oracle encoders, the oracle's
    reorder and decoders, the library's torch-facing encoder and its C entry point must reproduce them: bits,
    element types and shapes -- the serialised form a converted checkpoint has."""
    import ctypes
    import os
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", f"reference_format_{name}.npz"))
    w = g["w"]
    want = (g["compressed_val"], g["tile_offsets_global"], g["tile_offsets_median"], g["bitmap"])
    assert [str(a.dtype) for a in want] == ["uint32", "int32", "uint16", "uint64"]
    assert list(g["torch_dtypes"]) == ["torch.uint32", "torch.int32", "torch.uint16", "torch.uint64"]
    assert list(g["torch_shapes"]) == [str(tuple(a.shape)) for a in want]          # one-dimensional, as stored
    for enc in (O.encode(w), coracle.encode(w)):
        for got, ref in zip(enc, want):
            assert got.dtype == ref.dtype and got.shape == ref.shape and (got == ref).all()
    assert (O.reorder(w) == g["reordered"]).all() and (coracle.reorder(w) == g["reordered"]).all()
    assert (O.decode(*want, *w.shape) == w).all() and (coracle.decode(*want, *w.shape) == w).all()
    # the product: the call-site function (torch tensors of the reference's dtypes) and the C entry point under it
    prod = T.compress_weight(torch.from_numpy(w))
    _same(prod, want)
    assert [str(t.dtype) for t in prod] == list(g["torch_dtypes"])
    assert (T.reorder_weight(torch.from_numpy(w)).numpy() == g["reordered"]).all()
    lib = T._lib.load()
    n, k = w.shape
    sizes = [ctypes.c_int64() for _ in range(4)]
    assert lib.ternaspmm_encode_sizes(n, k, *[ctypes.byref(v) for v in sizes]) == 0
    bm = np.zeros(sizes[0].value, np.uint64)
    off = np.zeros(sizes[1].value, np.int32)
    med = np.zeros(sizes[2].value, np.uint16)
    vals = np.zeros(max(sizes[3].value, 1), np.uint32)
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    words = lib.ternaspmm_encode_i8(p(np.ascontiguousarray(w)), n, k, p(bm), p(off), p(med), p(vals))
    assert words == want[0].size and (vals[:words] == want[0]).all()
    assert (off == want[1]).all() and (med == want[2]).all() and (bm == want[3]).all()


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
