"""Pins the oracle's linear-layer arithmetic (no GPU).

  int8 family - the integer matmul is exact; with x == 1 and unit scales the output is the row
                sums of W, the construction the reference's own tests/test_kernel.cu:79-92 uses
                (glibc rand() without srand, reproduced here through libc);
                epilogue: C (volatile float, one operation at a time) == numpy float32, and the
                two rounding orders are shown to differ on some element (so a swapped formula fails)
  bf16 family - C fp64 loop == numpy fp64 matmul; linear in the scale; sign flip of W flips the output
  quantisers  - quant_input and quant_weight_int8 against answers worked by hand (ties to even, exact and
                inexact scales, the clamps), on both restatements and on the converter's own function
"""
import ctypes

import numpy as np
import pytest

from oracle import terna_oracle as O
from tests._util import make_bf16_activations, make_int8_activations, make_ternary


def glibc_rand_ternary(n, k, sparsity_pct):
    """W as tests/test_kernel.cu:83-91 builds it: r = rand()%100; nonzero iff r >= sparsity,
    then sign = (rand()%2)*2-1, row-major, from glibc's default seed."""
    libc = ctypes.CDLL("libc.so.6")
    libc.srand(1)                      # the state a program has when it never calls srand
    w = np.zeros((n, k), dtype=np.int8)
    for i in range(n):
        for j in range(k):
            if libc.rand() % 100 >= sparsity_pct:
                w[i, j] = (libc.rand() % 2) * 2 - 1
    return w


def test_x_equal_one_gives_row_sums(coracle):
    n, k, m = 64, 128, 8
    w = glibc_rand_ternary(n, k, 45)
    x = np.ones((m, k), dtype=np.int8)
    one = O.f32_to_bf16_bits(np.ones(4, np.float32))
    out = coracle.spmm_i8(x, w, one[:1].repeat(m), one, 4, 0)
    want = O.f32_to_bf16_bits(np.tile(w.sum(axis=1, dtype=np.int64).astype(np.float32), (m, 1)))
    assert (out == want).all()
    assert (O.spmm_i8(x, w, one[:1].repeat(m), one, 4, 0) == want).all()


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("n,ws_num", [(128, 1), (128, 2), (256, 4), (3840, 3), (3840, 1)])
def test_int8_epilogue_c_equals_numpy(coracle, mode, n, ws_num):
    k, m = 192, 5
    w = make_ternary(n, k, 0.4, 100 + n + ws_num)
    xq, s = make_int8_activations(m, k, 200 + n)
    ws = O.f32_to_bf16_bits(np.array([0.8125, 1.59375, 2.71875, 0.3359375], np.float32))
    a = coracle.spmm_i8(xq, w, s, ws, ws_num, mode)
    b = O.spmm_i8(xq, w, s, ws, ws_num, mode)
    assert (a == b).all()


def test_the_two_epilogue_orders_differ_somewhere(coracle):
    n, k, m = 256, 192, 16
    w = make_ternary(n, k, 0.4, 7)
    xq, s = make_int8_activations(m, k, 8)
    ws = O.f32_to_bf16_bits(np.array([1.59375], np.float32))
    a = coracle.spmm_i8(xq, w, s, ws, 1, 0)
    b = coracle.spmm_i8(xq, w, s, ws, 1, 1)
    assert (a != b).any()


def test_prefill_epilogue_zero_scale_gives_zero(coracle):
    n, k, m = 128, 64, 2
    w = make_ternary(n, k, 0.4, 9)
    xq, s = make_int8_activations(m, k, 10)
    s = s.copy()
    s[1] = 0
    ws = O.f32_to_bf16_bits(np.array([1.5], np.float32))
    out = coracle.spmm_i8(xq, w, s, ws, 1, 1)
    # float(acc) * 0 keeps acc's sign: the row is all +0.0 / -0.0
    assert not (out[1] & 0x7FFF).any() and out[0].any()


def test_prefill_group_is_per_128_column_tile():
    # N = 192, ws_num = 3: groups of 64 columns on the decode path; the prefill path looks only
    # at the first column of each 128-wide tile
    cols = np.arange(192)
    assert O.ws_group_decode(cols, 192, 3).tolist() == [0] * 64 + [1] * 64 + [2] * 64
    assert O.ws_group_prefill(cols, 192, 3).tolist() == [0] * 128 + [2] * 64
    assert O.ws_group_prefill(np.arange(3840), 3840, 1).max() == 0


def test_bf16_golden_c_equals_numpy_and_is_linear(coracle):
    n, k, m = 128, 256, 4
    w = make_ternary(n, k, 0.4, 11)
    x = make_bf16_activations(m, k, 12, outlier_frac=0.01)
    sc = np.array([0.7, 1.9], np.float32)
    a = coracle.spmm_bf16(x, w, sc, 2)
    b = O.spmm_bf16_golden(x, w, sc, 2)
    assert np.allclose(a, b, rtol=1e-12, atol=1e-9)
    assert np.allclose(coracle.spmm_bf16(x, -w, sc, 2), -a, rtol=0, atol=0)
    assert np.allclose(coracle.spmm_bf16(x, w, 2 * sc, 2), 2 * a, rtol=1e-15)


def test_quant_input_c_equals_numpy(coracle):
    x = make_bf16_activations(6, 320, 13, outlier_frac=0.02)
    q1, s1 = coracle.quant_input(x)
    q2, s2 = O.quant_input(x)
    assert (q1 == q2).all() and (s1 == s2).all()
    assert np.abs(q1).max() <= 127 and (np.abs(q1).max(axis=1) >= 126).all()


def _row(values, width=16):
    """One activation row: the given bf16-exact values, zero-padded."""
    r = np.zeros(width, np.float32)
    r[:len(values)] = values
    bits = O.f32_to_bf16_bits(r)
    assert (O.bf16_bits_to_f32(bits) == r).all(), "test vector must be exact in bf16"
    return bits


# Known answers of quant_input (model.py:120-123) worked by hand, for the three evaluations the reference's two lines
# admit (oracle: quant_input(x, mode)):
#   rounded  (this build's default) s = bf16(127 / max(max|x|, 1e-5)); q = clamp(round_half_even(fp32(x * s))), with
#            the ROUNDED s in the product;
#   compiled (the method as shipped, under @torch.compile) fp32 throughout: `127 / t` on a tensor is t.reciprocal() * 127,
#            so the multiplier is fl32(fl32(1 / max) * 127), UNROUNDED; s = its bf16;
#   eager    (no torch.compile, bf16 tensor) every op rounded to bf16: s = bf16(bf16(1 / max) * 127), product bf16(x * s).
# Each row is chosen so that one plausible mistake fails it.
# (values, s, q rounded, q compiled, q eager[, s eager]); None = as rounded.
QUANT_INPUT_KAT = [
    # max|x| = 127 -> s = 1 exactly, q = round_half_even(x): floor(x + 0.5) or round-half-away fails
    ([127.0, 0.5, 1.5, 2.5, -2.5, -0.5, 100.5, 101.5, -126.5, 3.5, -1.5],
     1.0, [127, 0, 2, 2, -2, 0, 100, 102, -126, 4, -2], None, None),
    # max|x| = 1 -> s = 127 (exact in bf16); 0.5 * 127 = 63.5 is a tie -> 64 (even), -63.5 -> -64
    ([1.0, -1.0, 0.5, -0.5, 0.25, 0.0078125, 0.00390625],
     127.0, [127, -127, 64, -64, 32, 1, 0], None, None),        # 31.75 -> 32, 0.992 -> 1, 0.496 -> 0
    # max|x| = 0.5 -> s = 254 (exact); max|x| = 4 -> s = 31.75 (exact): a missing or inverted scale fails
    ([0.5, -0.25, 0.125], 254.0, [127, -64, 32], None, None),   # -63.5 -> -64, 31.75 -> 32
    ([4.0, 2.0, -1.0, 0.0625], 31.75, [127, 64, -32, 2], None, None),   # 63.5 -> 64, -31.75 -> -32, 1.984 -> 2
    # max|x| = 129/128: 127 / (129/128) = 16256/129 = 126.01550..., s = 126 in bf16 (rounds DOWN).
    #   rounded : 0.75 * 126 = 94.5, a tie -> 94;  (129/256) * 126 = 63.49 -> 63
    #   compiled: fl32(128/129) = 2080895/2097152, times 127 -> t = 1032319/8192 = 126.0155029 (just below 16256/129);
    #             0.75 * t = 94.5116 -> 95;  (129/256) * t = 63.4999995, which is nearer to 63.5 than to the fp32
    #             number below it (63.5 - 2^-18) -> the fp32 product IS 63.5, a tie -> 64.  (An implementation that
    #             keeps the product in double gets 63.)
    #   eager   : bf16(128/129) = 0.9921875, times 127 = 126.008 -> s = 126; 0.75 * 126 = 94.5 is exact in bf16 -> 94;
    #             63.49 rounds to 63.5 in bf16 (step 0.25) -> 64
    ([1.0078125, 0.75, 0.50390625, -0.75], 126.0, [127, 94, 63, -94], [127, 95, 64, -95], [127, 94, 64, -94]),
    # max|x| = 255/128: 127 / 1.9921875 = 63.749 rounds UP to s = 63.75; max|x| * s = 127.002 -> 127:
    # the rounding of s can overshoot 127 by at most 127 * 2^-8 < 0.5, so the clamp never bites -- in fp32.  Eager mode
    # rounds the reciprocal first: 1 / 1.9921875 = 0.50196 -> bf16 0.50390625 (the upper neighbour, by 2e-5), times 127 =
    # 63.996 -> s = 64; then 1.9921875 * 64 = 127.5 exactly, a tie -> 128 -> clamped to 127, and -127.5 -> -128 stays
    ([1.9921875, -1.9921875, 1.0], 63.75, [127, -127, 64], None, [127, -128, 64], 64.0),
    # max|x| = 1 -> s = 127; x = 135/512: x * s = 33.486 -> 33 in fp32, but bf16 (step 0.25 between 32 and 64) rounds the
    # product to 33.5 first, a tie -> 34: only the eager evaluation rounds the product
    ([1.0, 0.263671875], 127.0, [127, 33], None, [127, 34]),
]
KAT_MODES = [(O.QUANT_ROUNDED, 2), (O.QUANT_COMPILED, 3), (O.QUANT_EAGER, 4)]


@pytest.mark.parametrize("row", QUANT_INPUT_KAT)
def test_quant_input_known_answers(coracle, row):
    values, s_want = row[0], row[1]
    x = _row(values).reshape(1, -1)
    for mode, col in KAT_MODES:
        q_want = row[col] if row[col] is not None else row[2]
        s_want = row[5] if mode == O.QUANT_EAGER and len(row) > 5 else row[1]
        for impl in (O.quant_input, coracle.quant_input):
            q, s = impl(x, mode)
            assert O.bf16_bits_to_f32(s).tolist() == [s_want]
            assert q[0, :len(q_want)].tolist() == q_want and not q[0, len(q_want):].any(), (mode, q[0].tolist())
    assert (O.quant_input(x)[0] == O.quant_input(x, O.QUANT_ROUNDED)[0]).all()      # the default is the rounded rule


def test_quant_input_call_site_function_known_answers():
    """ternainfer_amd.linear.quant_input -- what SpBitLinear / BF16BitLinear of this build call, written with torch ops
    as the reference's method is -- on the same rows, in the three modes (CPU tensors)."""
    import torch
    from ternainfer_amd import linear as L
    for row in QUANT_INPUT_KAT:
        x = torch.from_numpy(O.bf16_bits_to_f32(_row(row[0]).reshape(1, -1))).to(torch.bfloat16)
        for mode, col in KAT_MODES:
            q_want = row[col] if row[col] is not None else row[2]
            s_want = row[5] if mode == O.QUANT_EAGER and len(row) > 5 else row[1]
            q, s = L.quant_input(x, mode)
            assert q.dtype == torch.int8 and s.dtype == torch.bfloat16 and s.shape == (1, 1)
            assert float(s) == s_want and q[0, :len(q_want)].tolist() == q_want, (mode, q[0].tolist())


def test_quant_input_modes_on_random_rows(coracle):
    """The three evaluations agree with each other on most elements and never differ by more than two steps; the two
    restatements agree bit for bit in every mode; and the torch statement of the reference's own two lines, run
    eagerly on the bf16 tensor, IS the eager mode."""
    import torch
    x = make_bf16_activations(16, 2560, 77)
    got = {}
    for mode, _ in KAT_MODES:
        q1, s1 = O.quant_input(x, mode)
        q2, s2 = coracle.quant_input(x, mode)
        assert (q1 == q2).all() and (s1 == s2).all()
        got[mode] = q1.astype(np.int32)
    for a in got:
        for b in got:
            d = np.abs(got[a] - got[b])
            assert d.max() <= 2 and (a == b or 0.01 < (d != 0).mean() < 0.15), (a, b, d.max(), (d != 0).mean())
    xt = torch.from_numpy(O.bf16_bits_to_f32(x)).to(torch.bfloat16)
    s = 127 / xt.abs().max(dim=-1, keepdim=True).values.clamp_(min=1e-5)            # model.py:122-123, verbatim semantics
    q = (xt * s).round().clamp(-128, 127).to(torch.int8)
    assert (q.numpy() == got[O.QUANT_EAGER]).all()


def test_quant_input_all_zero_row(coracle):
    """max|x| = 0 is clamped to 1e-5: s = bf16(127 / 1e-5f) = bf16(12 700 000.3) = 1.515625 * 2^23
    (bits 0x4B42), q = 0."""
    x = np.zeros((1, 32), np.uint16)
    for impl in (O.quant_input, coracle.quant_input):
        q, s = impl(x)
        assert s.tolist() == [0x4B42] and O.bf16_bits_to_f32(s).tolist() == [1.515625 * 2.0 ** 23]
        assert not q.any()


def test_quant_input_rows_are_independent(coracle):
    """The scale is per row (dim=-1, keepdim): stacking KAT rows must not change any of them."""
    width = 16
    x = np.stack([_row(row[0], width) for row in QUANT_INPUT_KAT])
    for impl in (O.quant_input, coracle.quant_input):
        q, s = impl(x)
        assert O.bf16_bits_to_f32(s).tolist() == [row[1] for row in QUANT_INPUT_KAT]
        for r, row in enumerate(QUANT_INPUT_KAT):
            assert q[r, :len(row[2])].tolist() == row[2]


# Known answers of quant_weight_int8 (convert_TernaInfer.py:159-163): s = 1 / max(mean|W|, 1e-5),
# W_t = clamp(round_half_even(W * s), -1, 1), scale = 1 / s.
QUANT_WEIGHT_KAT = [
    # mean|W| = 1 -> s = 1: ties 0.5 -> 0, 1.5 -> 2 -> clamp 1, 2.5 -> 2 -> 1; floor(x + 0.5) turns 0.5 into 1
    ([0.5, -0.5, 1.5, -1.5, 0.25, 2.5, 0.75, 0.5], 1.0, [0, 0, 1, -1, 0, 1, 1, 0]),
    # mean|W| = 0.5 -> s = 2: 0.25 * 2 = 0.5 -> 0, 0.75 * 2 = 1.5 -> 2 -> 1; a max- or rms-based scale fails
    ([0.25, 0.75, -0.25, -0.75], 0.5, [0, 1, 0, -1]),
    # mean|W| = 2 -> s = 0.5: 1.0 * 0.5 = 0.5 -> 0, 3 * 0.5 = 1.5 -> 2 -> 1, -3 -> -1, 1.0078125 * 0.5 > 0.5 -> 1
    ([1.0, 3.0, -3.0, 1.0078125, 2.9921875, -1.0], 2.0, [0, 1, -1, 1, 1, 0]),
]


@pytest.mark.parametrize("values,scale_want,t_want", QUANT_WEIGHT_KAT)
def test_quant_weight_int8_known_answers(values, scale_want, t_want):
    import torch
    import ternainfer_amd as T
    w = np.array(values, np.float32).reshape(2, -1)
    assert np.abs(w).mean() == scale_want                       # the vector is built for an exact mean
    t, scale = O.quant_weight_int8(w)
    assert t.dtype == np.int8 and t.reshape(-1).tolist() == t_want and float(scale) == scale_want
    # the converter's own function (the reference's four lines on torch tensors) on the same vector, in fp32
    # and in bf16 (every value, product and the mean are exact in bf16 here)
    for dtype in (torch.float32, torch.bfloat16):
        tt, ss = T.quant_weight_int8(torch.from_numpy(w).to(dtype))
        assert tt.dtype == torch.int8 and tt.reshape(-1).tolist() == t_want
        assert ss.dtype == torch.bfloat16 and ss.shape == (1,) and float(ss) == scale_want


def test_quant_weight_int8_all_zero():
    t, scale = O.quant_weight_int8(np.zeros((4, 4), np.float32))
    assert not t.any() and abs(float(scale) - 1e-5) <= 1e-11   # the clamp of the mean


# ------------------------------------------------------------------ glue between two linears
def test_rmsnorm_closed_forms():
    """What the mathematics fixes for RMSNorm: a constant row maps to sign * weight, a power-of-two
    rescale of the row changes nothing when eps = 0, and a 4-element case equals the hand formula."""
    w = O.f32_to_bf16_bits(np.linspace(0.5, 2.0, 64, dtype=np.float32))
    ones = O.f32_to_bf16_bits(np.full((1, 64), -3.0, np.float32))
    assert (O.rmsnorm(ones, w, 0.0) == O.f32_to_bf16_bits(-O.bf16_bits_to_f32(w))).all()
    x = make_bf16_activations(5, 64, 71)
    x4 = O.f32_to_bf16_bits(O.bf16_bits_to_f32(x) * np.float32(4.0))
    assert (O.rmsnorm(x, w, 0.0) == O.rmsnorm(x4, w, 0.0)).all()
    v = np.array([[1.0, -2.0, 3.0, 0.5]], np.float32)
    want = v / np.sqrt((1 + 4 + 9 + 0.25) / 4 + 1e-5) * np.array([1.0, 0.5, 2.0, 1.0])
    got = O.bf16_bits_to_f32(O.rmsnorm(O.f32_to_bf16_bits(v), O.f32_to_bf16_bits(np.array([1.0, 0.5, 2.0, 1.0], np.float32)), 1e-5))
    assert (got == O.bf16_bits_to_f32(O.f32_to_bf16_bits(want.astype(np.float32)))).all()


def test_relu2_mul_and_residual_add_small_cases():
    x13 = O.f32_to_bf16_bits(np.array([[-1.0, 0.0, 1.5, 3.0, 2.0, 2.0, -2.0, 0.5]], np.float32))
    assert O.bf16_bits_to_f32(O.relu2_mul(x13)).tolist() == [[0.0, 0.0, -4.5, 4.5]]
    # 1 + 2^-8 is not a bf16 value: the sum rounds to even
    a = O.f32_to_bf16_bits(np.array([1.0], np.float32))
    b = O.f32_to_bf16_bits(np.array([2.0 ** -8], np.float32))
    assert O.bf16_bits_to_f32(O.residual_add(a, b)).tolist() == [1.0]
    c = O.f32_to_bf16_bits(np.array([3 * 2.0 ** -8], np.float32))
    assert O.bf16_bits_to_f32(O.residual_add(a, c)).tolist() == [1.0 + 2.0 ** -6]


def test_rope_and_attention_closed_forms():
    """Angle 0 is the identity, angle pi/2 maps (x1, x2) to (-x2, x1); attention over identical value
    rows returns that row, and a key that dominates the softmax returns its value row."""
    x = make_bf16_activations(3, 64, 81)
    zero, one = np.zeros((3, 32), np.float32), np.ones((3, 32), np.float32)
    assert (O.rope_rotate_half(x, one, zero) == x).all()
    xf = O.bf16_bits_to_f32(x)
    want = np.concatenate([-xf[:, 32:], xf[:, :32]], axis=-1)
    assert (O.bf16_bits_to_f32(O.rope_rotate_half(x, zero, one)) == want).all()
    # adjacent pairing: the same rotation after moving the pairs (2j, 2j+1) to (j, j+D/2); norm of a pair kept
    rng = np.random.default_rng(86)
    ang = rng.uniform(-3, 3, (3, 32)).astype(np.float32)
    cos, sin = np.cos(ang), np.sin(ang)
    de = np.concatenate([x[:, 0::2], x[:, 1::2]], axis=-1)
    rot = O.rope_rotate_half(de, cos, sin)
    back = np.empty_like(rot)
    back[:, 0::2], back[:, 1::2] = rot[:, :32], rot[:, 32:]
    assert (O.rope_adjacent(x, cos, sin) == back).all()
    assert (O.rope_adjacent(x, one, zero) == x).all()
    sw = np.empty_like(xf)
    sw[:, 0::2], sw[:, 1::2] = -xf[:, 1::2], xf[:, 0::2]
    assert (O.bf16_bits_to_f32(O.rope_adjacent(x, zero, one)) == sw).all()
    q = make_bf16_activations(2 * 4, 64, 82).reshape(2, 4, 64)
    k = make_bf16_activations(2 * 2 * 10, 64, 83).reshape(2, 2, 10, 64)
    v = np.broadcast_to(make_bf16_activations(1, 64, 84), (2, 2, 10, 64)).copy()
    got = O.attention_one_token(q, k, v, 7, 0.125)
    assert np.allclose(got, np.broadcast_to(O.bf16_bits_to_f32(v[0, 0, 0]), got.shape), rtol=0, atol=1e-12)
    k2 = np.zeros((1, 1, 5, 64), np.uint16)
    k2[0, 0, 3] = O.f32_to_bf16_bits(np.full(64, 8.0, np.float32))
    q2 = O.f32_to_bf16_bits(np.full((1, 1, 64), 8.0, np.float32))
    v2 = make_bf16_activations(5, 64, 85).reshape(1, 1, 5, 64)
    assert np.allclose(O.attention_one_token(q2, k2, v2, 5, 1.0)[0, 0], O.bf16_bits_to_f32(v2[0, 0, 3]), atol=1e-9)
    assert not np.allclose(O.attention_one_token(q2, k2, v2, 3, 1.0)[0, 0], O.bf16_bits_to_f32(v2[0, 0, 3]), atol=1e-3)


# ------------------------------------------------------------------ the glue functions against library routines
def test_attention_against_torch_sdpa():
    """attention_one_token / attention_new_tokens against torch.nn.functional.scaled_dot_product_attention in float64,
    at the 2B head layout (20 query heads on 5 kv heads, head size 128) with a scale that is not the default and
    values that differ per kv head: a wrong softmax scale, a wrong head -> kv-head mapping (h % KV instead of
    h // (H / KV)) or an off-by-one in the causal prefix each fail here."""
    import torch
    from torch.nn import functional as F
    b, h, kv, d, s_max, n = 2, 20, 5, 128, 48, 37
    scale = 0.0713
    q = make_bf16_activations(b * h, d, 301).reshape(b, h, d)
    k = make_bf16_activations(b * kv * s_max, d, 302).reshape(b, kv, s_max, d)
    v = make_bf16_activations(b * kv * s_max, d, 303).reshape(b, kv, s_max, d)
    t64 = lambda a: torch.from_numpy(O.bf16_bits_to_f32(a).astype(np.float64))
    rep = h // kv
    kk, vv = t64(k)[:, :, :n].repeat_interleave(rep, dim=1), t64(v)[:, :, :n].repeat_interleave(rep, dim=1)
    want = F.scaled_dot_product_attention(t64(q)[:, :, None], kk, vv, scale=scale)[:, :, 0].numpy()
    got = O.attention_one_token(q, k, v, n, scale)
    assert np.abs(got - want).max() < 1e-12
    wrong_scale = F.scaled_dot_product_attention(t64(q)[:, :, None], kk, vv)[:, :, 0].numpy()      # d ** -0.5
    assert np.abs(got - wrong_scale).max() > 1e-2
    kk_mod = t64(k)[:, :, :n].repeat(1, rep, 1, 1)                                                  # head h -> kv head h % KV
    vv_mod = t64(v)[:, :, :n].repeat(1, rep, 1, 1)
    wrong_map = F.scaled_dot_product_attention(t64(q)[:, :, None], kk_mod, vv_mod, scale=scale)[:, :, 0].numpy()
    assert np.abs(got - wrong_map).max() > 1e-2

    # several new tokens at slots first .. first + T - 1 of a cache that already holds `first` rows
    t_new, first = 9, 20
    qn = make_bf16_activations(b * h * t_new, d, 304).reshape(b, h, t_new, d)
    pos = np.arange(first, first + t_new)
    seen = torch.arange(s_max)[None, :] <= torch.from_numpy(pos)[:, None]                          # [T, S]
    kk, vv = t64(k).repeat_interleave(rep, dim=1), t64(v).repeat_interleave(rep, dim=1)
    want = F.scaled_dot_product_attention(t64(qn), kk, vv, attn_mask=seen[None, None], scale=scale).transpose(1, 2).numpy()
    got = O.attention_new_tokens(qn, k, v, pos, scale)                                             # [B, T, H, D]
    assert got.shape == want.shape and np.abs(got - want).max() < 1e-12
    off_by_one = torch.arange(s_max)[None, :] < torch.from_numpy(pos)[:, None]
    wrong = F.scaled_dot_product_attention(t64(qn), kk, vv, attn_mask=off_by_one[None, None], scale=scale).transpose(1, 2).numpy()
    assert np.abs(got - wrong).max() > 1e-2


def test_rmsnorm_against_torch_rms_norm():
    """rmsnorm against torch.nn.functional.rms_norm evaluated in float64 and rounded once to bf16: identical bits."""
    import torch
    from torch.nn import functional as F
    x = make_bf16_activations(7, 2560, 311, outlier_frac=0.01)
    w = O.f32_to_bf16_bits(np.random.default_rng(312).uniform(0.5, 1.5, 2560).astype(np.float32))
    for eps in (1e-5, 1e-2):
        ref = F.rms_norm(torch.from_numpy(O.bf16_bits_to_f32(x).astype(np.float64)), (2560,),
                         torch.from_numpy(O.bf16_bits_to_f32(w).astype(np.float64)), eps)
        want = O.f32_to_bf16_bits(ref.numpy().astype(np.float32))
        assert (O.rmsnorm(x, w, eps) == want).all()
    assert (O.rmsnorm(x, w, 1e-5) != O.rmsnorm(x, w, 1e-2)).any()          # eps takes part


def test_rope_against_complex_multiplication():
    """Both pairings are the complex product (x1 + i x2) * exp(i angle) per pair, rounded once to bf16: compared with
    numpy's complex128 product (the oracle's fp32 products and sums stay within one bf16 step of it, and agree on
    all but a sliver of the elements); a conjugated angle or swapped cos / sin fails by far more."""
    rng = np.random.default_rng(321)
    x = make_bf16_activations(6, 128, 322)
    ang = rng.uniform(-np.pi, np.pi, (6, 64))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    xf = O.bf16_bits_to_f32(x).astype(np.float64)
    rot = np.exp(1j * np.arctan2(sin.astype(np.float64), cos.astype(np.float64)))

    def key(bits):
        bits = bits.astype(np.int32)
        return np.where(bits & 0x8000, -(bits & 0x7FFF), bits & 0x7FFF)

    z = (xf[:, 0::2] + 1j * xf[:, 1::2]) * rot
    want = np.empty_like(xf)
    want[:, 0::2], want[:, 1::2] = z.real, z.imag
    d = np.abs(key(O.rope_adjacent(x, cos, sin)) - key(O.f32_to_bf16_bits(want.astype(np.float32))))
    assert d.max() <= 1 and (d != 0).mean() < 0.01
    conj = np.abs(key(O.rope_adjacent(x, cos, -sin)) - key(O.f32_to_bf16_bits(want.astype(np.float32))))
    swapped = np.abs(key(O.rope_adjacent(x, sin, cos)) - key(O.f32_to_bf16_bits(want.astype(np.float32))))
    assert conj.max() > 64 and swapped.max() > 64
    z = (xf[:, :64] + 1j * xf[:, 64:]) * rot
    want = np.concatenate([z.real, z.imag], axis=-1)
    d = np.abs(key(O.rope_rotate_half(x, cos, sin)) - key(O.f32_to_bf16_bits(want.astype(np.float32))))
    assert d.max() <= 1 and (d != 0).mean() < 0.01
