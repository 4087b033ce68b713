"""Pins the CPU oracle's restatement of the weight format (no GPU, no reference import).

What fixes each part:
  reorder   - bijection on a 16x16 block, closed form == branch form (two source statements of
              the reference), and the consumer replay below
  encode    - closed-form tiles (all zero / all +1 / all -1 / one nonzero), stream invariants,
              C loop form == numpy closed form, and the consumer replay
  consumer  - oracle_consumer_sim replays the reference kernel's lane-level fragment build
              (MatMulUtilities.cuh:79-114) on the encoded stream and must hand every lane the
              mma.m16n8k16 A fragment of the ORIGINAL matrix; a wrong traversal order, bit
              position, sign polarity or median offset breaks it
  decode    - round trip and brute force
"""
import numpy as np
import pytest

from oracle import terna_oracle as O
from tests._util import make_row_skewed, make_ternary


def test_reorder_is_bijection_and_matches_branch_form(coracle):
    di, dk = O.reorder_index_maps()
    flat = di * 16 + dk
    assert sorted(flat.reshape(-1).tolist()) == list(range(256))
    w = np.arange(256, dtype=np.int16).reshape(16, 16)
    w8 = (w % 127).astype(np.int8)
    assert (coracle.reorder(w8) == O.reorder(w8)).all()
    # a labelled block: element (i,k) must land at (dst_i, dst_k)
    lab = np.zeros((16, 16), dtype=np.int8)
    for i in range(16):
        for k in range(16):
            lab[:] = 0
            lab[i, k] = 1
            r = coracle.reorder(lab)
            assert r[di[i, k], dk[i, k]] == 1 and r.sum() == 1


def test_reorder_inverse_closed_form():
    di, dk = O.reorder_index_maps()
    for i in range(16):
        for k in range(16):
            ri, rk = di[i, k], dk[i, k]
            assert (ri & 7) + 8 * (rk >> 3) == i
            assert 4 * ((rk & 7) >> 1) + 2 * (ri >> 3) + (rk & 1) == k


@pytest.mark.parametrize("enc", ["c", "np"])
def test_closed_form_tiles(coracle, enc):
    encode = coracle.encode if enc == "c" else O.encode
    # all zero: nothing in the stream
    vals, off, med, bm = encode(np.zeros((64, 128), dtype=np.int8))
    assert vals.size == 0 and off.tolist() == [0, 0, 0] and med.tolist() == [0] * 6 and not bm.any()
    # all +1: full bitmaps, 4096 signs per tile, all sign bits clear
    vals, off, med, bm = encode(np.ones((64, 128), dtype=np.int8))
    assert off.tolist() == [0, 4096, 8192] and med.tolist() == [1024, 2048, 3072] * 2
    assert (bm == np.uint64(0xFFFFFFFFFFFFFFFF)).all() and vals.size == 256 and not vals.any()
    # all -1: same, all sign bits set
    vals, off, med, bm = encode(-np.ones((64, 64), dtype=np.int8))
    assert off.tolist() == [0, 4096] and (vals == np.uint32(0xFFFFFFFF)).all() and vals.size == 128


@pytest.mark.parametrize("enc", ["c", "np"])
def test_single_nonzero_position(coracle, enc):
    """One nonzero at (row, col): exactly one bit, where the format's index algebra says."""
    encode = coracle.encode if enc == "c" else O.encode
    rng = np.random.default_rng(7)
    for _ in range(64):
        row, col = int(rng.integers(0, 128)), int(rng.integers(0, 192))
        sign = -1 if rng.random() < 0.5 else 1
        w = np.zeros((128, 192), dtype=np.int8)
        w[row, col] = sign
        vals, off, med, bm = encode(w)
        tile = (row // 64) * 3 + col // 64
        band, g = (row % 64) // 16, (col % 64) // 16
        i, k = row % 16, col % 16
        sk, r = i >> 3, i & 7                 # row half -> which column-half of the permuted block
        sm, c = (k >> 1) & 1, 2 * (k >> 2) + (k & 1)
        idx = tile * 64 + band * 16 + g * 4 + 2 * sk + sm
        assert bm[idx] == np.uint64(1) << np.uint64(8 * r + c)
        assert np.count_nonzero(bm) == 1
        assert vals.size == 1 and vals[0] == (1 if sign < 0 else 0)
        d = np.diff(off)
        assert d[tile] == 32 and d.sum() == 32
        want_med = [0 if b < band else 1 for b in range(3)]
        assert med[3 * tile:3 * tile + 3].tolist() == want_med


@pytest.mark.parametrize("shape,p0,seed", [((64, 64), 0.45, 1), ((128, 192), 0.40, 2), ((256, 128), 0.05, 3),
                                           ((192, 320), 0.97, 4)])
def test_c_and_numpy_encoders_agree_and_invariants_hold(coracle, shape, p0, seed):
    w = make_ternary(*shape, p0, seed)
    a = coracle.encode(w)
    b = O.encode(w)
    for x, y in zip(a, b):
        assert x.dtype == y.dtype and x.shape == y.shape and (x == y).all()
    vals, off, med, bm = a
    assert vals.dtype == np.uint32 and off.dtype == np.int32 and med.dtype == np.uint16 and bm.dtype == np.uint64
    ntiles = shape[0] * shape[1] // 4096
    pc = np.array([bin(int(v)).count("1") for v in bm]).reshape(ntiles, 64).sum(axis=1)
    d = np.diff(off)
    assert (off % 32 == 0).all() and (d >= pc).all() and (d - pc < 32).all()
    assert pc.sum() == np.count_nonzero(w) and vals.size == off[-1] // 32
    # median offsets = cumulative unpadded counts of bands 0..2
    band_pc = np.array([bin(int(v)).count("1") for v in bm]).reshape(ntiles, 4, 16).sum(axis=2)
    assert (med.reshape(ntiles, 3) == np.cumsum(band_pc, axis=1)[:, :3]).all()


@pytest.mark.parametrize("shape,p0,seed", [((64, 64), 0.45, 11), ((128, 192), 0.40, 12), ((64, 256), 0.0, 13)])
def test_reference_consumer_replay_recovers_original_matrix(coracle, shape, p0, seed):
    w = make_ternary(*shape, p0, seed)
    enc = coracle.encode(w)
    tiles_k = shape[1] // 64
    for tile in range(shape[0] * shape[1] // 4096):
        for band in range(4):
            blk = coracle.consumer_sim(*enc, tile, band)
            r0 = (tile // tiles_k) * 64 + band * 16
            c0 = (tile % tiles_k) * 64
            assert (blk == w[r0:r0 + 16, c0:c0 + 64]).all(), (tile, band)


@pytest.mark.parametrize("make", ["iid", "skewed", "dense", "empty"])
def test_round_trip(coracle, make):
    n, k = 128, 192
    w = {"iid": lambda: make_ternary(n, k, 0.4, 21), "skewed": lambda: make_row_skewed(n, k, 22),
         "dense": lambda: make_ternary(n, k, 0.0, 23), "empty": lambda: np.zeros((n, k), np.int8)}[make]()
    enc = coracle.encode(w)
    assert (coracle.decode(*enc, n, k) == w).all()
    assert (O.decode(*enc, n, k) == w).all()


def test_decode_detects_corrupt_median_offset(coracle):
    w = make_ternary(64, 64, 0.4, 31)
    vals, off, med, bm = coracle.encode(w)
    med = med.copy()
    med[1] += 1
    with pytest.raises(ValueError):
        coracle.decode(vals, off, med, bm, 64, 64)


def test_bf16_rounding_helpers(coracle):
    x = np.array([1.0, 1.00390625, 1.01171875, -2.5, 3.3895314e38, 1e-40, 0.0], dtype=np.float32)
    want = [coracle.lib.oracle_f32_to_bf16(float(v)) for v in x]
    assert O.f32_to_bf16_bits(x).tolist() == want
    # ties to even: 1 + 2^-8 is halfway between 1.0 (even mantissa) and 1 + 2^-7
    assert O.f32_to_bf16_bits(np.array([1.00390625], np.float32))[0] == 0x3F80
    assert O.f32_to_bf16_bits(np.array([1.01171875], np.float32))[0] == 0x3F82


def test_p2_pack_round_trip_and_field_positions():
    """The library's load-time layout: unpack(pack(W)) == W, and one weight at (row, col) sets
    exactly the 2-bit field the layout definition names."""
    w = make_ternary(128, 192, 0.4, 51)
    p = O.pack_p2(w)
    assert p.shape == (8, 3, 64) and p.dtype == np.uint32 and (O.unpack_p2(p, 128, 192) == w).all()
    rng = np.random.default_rng(52)
    for _ in range(64):
        row, col = int(rng.integers(0, 128)), int(rng.integers(0, 192))
        sign = -1 if rng.random() < 0.5 else 1
        one = np.zeros((128, 192), np.int8)
        one[row, col] = sign
        p = O.pack_p2(one)
        j = col & 15
        bit = 8 * (j & 3) + 2 * (j >> 2)
        want = np.zeros_like(p)
        want[row >> 4, col >> 6, 4 * (row & 15) + ((col >> 4) & 3)] = (3 if sign < 0 else 1) << bit
        assert (p == want).all()
