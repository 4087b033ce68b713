"""CPU oracle for the TernaSpMM path -- TEST INFRASTRUCTURE ONLY.

Two independent restatements of the reference's weight format live here:

* the C one (``terna_oracle.c``, loaded through ctypes by :class:`COracle`), written
  in the reference's loop order, and
* the numpy one below, written from the closed-form index algebra.

Tests cross-check them against each other, against closed-form tiles, and against a
replay of the reference kernel's own consumer (``consumer_sim``).  Only ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import this
module; the shipped package never does.

Reference files restated (paths relative to the reference checkout):
  convert/convert_utils.py:9-49, 52-228      reorder_weight / compress_weight
  kernels/TernaSpMM.cu:241-439               reorder_WT_h / convert_reorderd
  kernels/src/SpMM/Reduction_Kernel.cuh:23-63          decode epilogue
  kernels/src/GEMM/epilogue_visitor_scale_ws.h:135-210 prefill epilogue
  convert/convert_TernaInfer.py:159-194      weight ternarisation and scale packing
  model.py:120-123                           activation quantisation

Parity status: every function is pinned by a test in tests/test_oracle_*.py --
``quant_input`` and ``quant_weight_int8`` by answers worked by hand (ties to even, scales
that are exact / round down / round up in bf16, the clamps; tests/test_oracle_linear.py).
``quant_input`` fixes one definition where the reference's two execution modes differ
(eager multiplies in the tensor's dtype, the compiled graph in fp32): fp32 product with
the bf16-rounded s, the s the epilogue divides by.  Except ``rmsnorm``, ``rope_rotate_half``,
``rope_adjacent`` and ``attention_one_token``: the reference takes RMSNorm, rope_padded
and the attention forward from xformers.ops (model.py:16), a third-party dependency that
is not part of the reference checkout and not installed here, so "parity unpinned"; the
formulas (y = x * rsqrt(mean(x^2) + eps) * weight, fp32 inside and one rounding to the
tensor's dtype; rotation of dimension pairs by position-dependent angles; softmax(q K^T
scale) V over the valid cache slots) restate those operators' published definitions and
are checked against what the mathematics fixes (tests/test_oracle_linear.py).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libterna_oracle.so")


# --------------------------------------------------------------------------- bf16 helpers
def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 storage (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    if np.any(nan):
        r = np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# --------------------------------------------------------------------------- reorder (closed form)
def reorder_index_maps():
    """For a 16x16 block return (dst_i, dst_k) as functions of source (i, k).

    Closed form of convert_utils.py:16-35 / TernaSpMM.cu:243-279:
        dst_i = (i & 7) + 8*((k >> 1) & 1)
        dst_k = 8*(i >> 3) + 2*(k >> 2) + (k & 1)
    """
    i, k = np.meshgrid(np.arange(16), np.arange(16), indexing="ij")
    return (i & 7) + 8 * ((k >> 1) & 1), 8 * (i >> 3) + 2 * (k >> 2) + (k & 1)


def reorder(w: np.ndarray) -> np.ndarray:
    """Apply the 16x16 block permutation to an [N, K] int8 matrix."""
    n, k = w.shape
    assert n % 16 == 0 and k % 16 == 0
    di, dk = reorder_index_maps()
    blocks = w.reshape(n // 16, 16, k // 16, 16)
    out = np.empty_like(blocks)
    out[:, di, :, dk] = blocks.transpose(1, 3, 0, 2)
    return out.reshape(n, k)


# --------------------------------------------------------------------------- encode (closed form)
def _stream_coordinates(n: int, k: int):
    """For every element (row, col) of the ORIGINAL matrix return
    (bitmap_index, bit) -- where the encoder puts it.

    tile T = (row//64)*(K/64) + col//64            convert_utils.py:96-97
    band   = (row % 64) // 16                      :110
    g      = (col % 64) // 16                      :119-120
    i, kk  = row % 16, col % 16; reorder -> (i', k')
    sm, sk = i' // 8, k' // 8; q = 2*sk + sm       :122-125 (column-major 2x2)
    bit    = (i' % 8)*8 + (k' % 8)                 :155-156
    """
    row, col = np.meshgrid(np.arange(n), np.arange(k), indexing="ij")
    tile = (row // 64) * (k // 64) + col // 64
    band = (row % 64) // 16
    g = (col % 64) // 16
    i, kk = row % 16, col % 16
    ri = (i & 7) + 8 * ((kk >> 1) & 1)
    rk = 8 * (i >> 3) + 2 * (kk >> 2) + (kk & 1)
    q = 2 * (rk >> 3) + (ri >> 3)
    bit = (ri & 7) * 8 + (rk & 7)
    bm = tile * 64 + band * 16 + g * 4 + q
    return bm, bit


def encode(w: np.ndarray):
    """Encode an ORIGINAL (not reordered) ternary int8 [N, K] matrix.

    Returns (compressed_val u32, TileOffsets_global i32, TileOffsets_median u16, bitmap u64),
    the tuple order of convert_utils.py:228.
    """
    w = np.ascontiguousarray(w, dtype=np.int8)
    n, k = w.shape
    assert n % 64 == 0 and k % 64 == 0
    ntiles = n * k // 4096
    bm, bit = _stream_coordinates(n, k)
    nz = w != 0
    bitmap = np.zeros(n * k // 64, dtype=np.uint64)
    np.bitwise_or.at(bitmap, bm[nz], np.uint64(1) << bit[nz].astype(np.uint64))

    # stream order: ascending (bitmap index, bit)
    key = (bm[nz].astype(np.int64) << 6) | bit[nz]
    order = np.argsort(key, kind="stable")
    neg = (w[nz] < 0)[order]
    tile_of = (key[order] >> 12)                      # 64 bitmaps * 64 bits per tile
    band_of = (key[order] >> 10) & 3

    cnt_tb = np.zeros((ntiles, 4), dtype=np.int64)
    np.add.at(cnt_tb, (tile_of, band_of), 1)
    per_tile = cnt_tb.sum(axis=1)
    padded = (per_tile + 31) // 32 * 32
    tile_off = np.zeros(ntiles + 1, dtype=np.int64)
    np.cumsum(padded, out=tile_off[1:])
    median = np.cumsum(cnt_tb, axis=1)[:, :3].astype(np.uint16).reshape(-1)

    # position of every nonzero in the padded stream
    start_unpadded = np.zeros(ntiles + 1, dtype=np.int64)
    np.cumsum(per_tile, out=start_unpadded[1:])
    rank = np.arange(order.size) - start_unpadded[tile_of]
    pos = tile_off[tile_of] + rank
    words = np.zeros(int(tile_off[-1]) // 32, dtype=np.uint32)
    np.bitwise_or.at(words, pos[neg] >> 5, (np.uint32(1) << (pos[neg] & 31).astype(np.uint32)))
    return words, tile_off.astype(np.int32), median, bitmap


def decode(compressed_val, tile_off, median_off, bitmap, n: int, k: int) -> np.ndarray:
    """Inverse of :func:`encode` -> ORIGINAL ternary int8 [N, K]."""
    bm, bit = _stream_coordinates(n, k)
    bitmap = np.asarray(bitmap, dtype=np.uint64)
    nz = ((bitmap[bm] >> bit.astype(np.uint64)) & np.uint64(1)).astype(bool)
    key = (bm[nz].astype(np.int64) << 6) | bit[nz]
    order = np.argsort(key, kind="stable")
    tile_of = key[order] >> 12
    ntiles = n * k // 4096
    per_tile = np.bincount(tile_of, minlength=ntiles)
    start_unpadded = np.zeros(ntiles + 1, dtype=np.int64)
    np.cumsum(per_tile, out=start_unpadded[1:])
    pos = np.asarray(tile_off, dtype=np.int64)[tile_of] + np.arange(order.size) - start_unpadded[tile_of]
    words = np.asarray(compressed_val, dtype=np.uint32)
    neg = ((words[pos >> 5] >> (pos & 31).astype(np.uint32)) & 1).astype(bool)
    vals = np.where(neg, -1, 1).astype(np.int8)
    out = np.zeros((n, k), dtype=np.int8)
    rows, cols = np.nonzero(nz)
    out[rows[order], cols[order]] = vals
    return out


# --------------------------------------------------------------------------- packed (load-time repack) layout
def pack_p2(w: np.ndarray) -> np.ndarray:
    """Dense ternary [N, K] -> the library's load-time layout "P2" (no counterpart in the reference).

    uint32 packed[N/16][K/64][64]; element [band][gk][4*i + g] holds the 16 weights of row
    16*band + i, columns 64*gk + 16*g .. +15, two bits each (bit0 = nonzero, bit1 = negative).
    Column j of the group sits at bit 8*(j & 3) + 2*(j >> 2): byte j & 3, 2-bit field j >> 2.  The 16
    weights of a word are the two bitmap bytes (sm = 0, 1) that one lane of the reference kernel
    decodes, so a repack from the reference format never moves a weight across lanes."""
    w = np.ascontiguousarray(w, dtype=np.int8)
    n, k = w.shape
    assert n % 16 == 0 and k % 64 == 0
    code = ((w != 0).astype(np.uint32) | ((w < 0).astype(np.uint32) << 1))
    j = np.arange(16)
    shift = (8 * (j & 3) + 2 * (j >> 2)).astype(np.uint32)
    blocks = code.reshape(n // 16, 16, k // 64, 4, 16)                # band, i, gk, g, q
    words = np.bitwise_or.reduce(blocks << shift, axis=-1)            # band, i, gk, g
    return np.ascontiguousarray(words.transpose(0, 2, 1, 3)).reshape(n // 16, k // 64, 64).astype(np.uint32)


def unpack_p2(packed: np.ndarray, n: int, k: int) -> np.ndarray:
    """Inverse of :func:`pack_p2`."""
    words = np.asarray(packed, dtype=np.uint32).reshape(n // 16, k // 64, 16, 4)   # band, gk, i, g
    j = np.arange(16)
    shift = (8 * (j & 3) + 2 * (j >> 2)).astype(np.uint32)
    code = (words[..., None] >> shift) & 3                                            # band, gk, i, g, q
    val = np.where(code & 1, np.where(code & 2, -1, 1), 0).astype(np.int8)
    return np.ascontiguousarray(val.transpose(0, 2, 1, 3, 4)).reshape(n, k)


# --------------------------------------------------------------------------- scales / quantisation
def ws_group_decode(cols: np.ndarray, n: int, ws_num: int) -> np.ndarray:
    """Reduction_Kernel.cuh:46-54."""
    cols = np.asarray(cols)
    if ws_num == 3 and n == 3840:
        return np.where(cols < 2560, 0, np.where(cols < 3200, 1, 2))
    return cols // (n // ws_num)


def ws_group_prefill(cols: np.ndarray, n: int, ws_num: int) -> np.ndarray:
    """epilogue_visitor_scale_ws.h:135-148 (group of the 128-column tile's first column)."""
    c0 = (np.asarray(cols) // 128) * 128
    if n == 3840:
        g = np.where(c0 < 2560, 0, np.where(c0 < 3200, 1, 2))
    else:
        g = c0 // (n // ws_num)
    return np.minimum(g, ws_num - 1)


def spmm_i8(x_q: np.ndarray, w: np.ndarray, s_bits: np.ndarray, ws_bits: np.ndarray,
            ws_num: int, mode: int, cols: np.ndarray | None = None) -> np.ndarray:
    """Integer matmul + reference epilogue -> bf16 storage [M, N].

    mode 0: bf16((float(acc)/s)*ws)      Reduction_Kernel.cuh:60
    mode 1: bf16(float(acc)*(ws/s)), coefficient 0 where s == 0   epilogue_visitor_scale_ws.h:188-205
    `cols`: only these output columns (weight-scale groups still follow the full N) -> [M, len(cols)];
    keeps the host matmul small at the largest shapes.
    """
    m, _ = x_q.shape
    n = w.shape[0]
    cols = np.arange(n) if cols is None else np.asarray(cols)
    # integer matmul through fp64 BLAS: exact while |acc| < 2^53 (here |acc| <= 128*K)
    acc = np.rint(x_q.astype(np.float64) @ w[cols].astype(np.float64).T).astype(np.int64)
    assert np.abs(acc).max(initial=0) < 2 ** 24
    accf = acc.astype(np.float32)
    s = bf16_bits_to_f32(s_bits).reshape(m, 1).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        if mode == 0:
            wsv = bf16_bits_to_f32(ws_bits)[ws_group_decode(cols, n, ws_num)].reshape(1, -1)
            r = (accf / s).astype(np.float32) * wsv.astype(np.float32)
        else:
            wsv = bf16_bits_to_f32(ws_bits)[ws_group_prefill(cols, n, ws_num)].reshape(1, -1)
            coeff = np.where(s != 0, (wsv / s).astype(np.float32), np.float32(0)).astype(np.float32)
            r = accf * coeff
    return f32_to_bf16_bits(r.astype(np.float32))


def spmm_bf16_golden(x_bits: np.ndarray, w: np.ndarray, scale: np.ndarray, ws_num: int) -> np.ndarray:
    """fp64 golden of the bf16-activation family: (X @ W^T) * scale[g(n)] -> float64 [M, N]."""
    x = bf16_bits_to_f32(x_bits).astype(np.float64)
    n = w.shape[0]
    acc = x @ w.astype(np.float64).T
    sc = np.asarray(scale, dtype=np.float32).astype(np.float64)[ws_group_decode(np.arange(n), n, ws_num)]
    return acc * sc.reshape(1, n)


QUANT_ROUNDED, QUANT_COMPILED, QUANT_EAGER = 0, 1, 2


def quant_input(x_bits: np.ndarray, mode: int = QUANT_ROUNDED):
    """model.py:120-123.  The reference's two lines leave the intermediate precision to PyTorch; `mode` says which
    evaluation is restated (see terna_oracle.c):
      QUANT_ROUNDED   fp32 compute, s = bf16(127 / max) and that rounded s multiplies (this build's default);
      QUANT_COMPILED  the @torch.compile'd method: fp32 compute without intermediate roundings to bf16.  `127 / t` on a
                      tensor is Tensor.__rtruediv__ = t.reciprocal() * 127, so the multiplier is fl32(fl32(1 / max) * 127),
                      unrounded; the returned s is its bf16 rounding;
      QUANT_EAGER     eager mode on a bf16 tensor, every op rounded to bf16: the clamp floor bf16(1e-5),
                      s = bf16(bf16(1 / max) * 127), and the product bf16(x * s) before round()."""
    x = bf16_bits_to_f32(x_bits)
    rb = lambda v: bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(v, dtype=np.float32)))
    floor = rb(np.float32(1e-5)) if mode == QUANT_EAGER else np.float32(1e-5)
    amax = np.maximum(np.abs(x).max(axis=-1, keepdims=True), floor).astype(np.float32)
    if mode == QUANT_ROUNDED:
        t = (np.float32(127.0) / amax).astype(np.float32)
    else:
        r = (np.float32(1.0) / amax).astype(np.float32)
        if mode == QUANT_EAGER:
            r = rb(r)
        t = (r * np.float32(127.0)).astype(np.float32)
    s_bits = f32_to_bf16_bits(t)
    mul = t if mode == QUANT_COMPILED else bf16_bits_to_f32(s_bits)
    prod = (x * mul).astype(np.float32)
    if mode == QUANT_EAGER:
        prod = rb(prod)
    q = np.clip(np.rint(prod), -128, 127).astype(np.int8)
    return q, s_bits.reshape(-1)


def bf16_bitlinear_golden(x_bits: np.ndarray, w_dense_bits: np.ndarray) -> np.ndarray:
    """model.py:135-153 (BF16BitLinear.forward, the reference's dense golden mode): quant_input, then
    F.linear(x_q as bf16, W) / s with W = ternary * scale stored dense in bf16 (convert_TernaInfer.py:112-114).
    Evaluated in float64 -> [M, N]; a composition of quant_input (pinned by known answers) and a float64
    matmul, so the reference's two bf16 roundings (GEMM output, quotient) show up as tolerance in the caller."""
    q, s_bits = quant_input(x_bits)
    w = bf16_bits_to_f32(w_dense_bits).astype(np.float64)
    s = bf16_bits_to_f32(s_bits).astype(np.float64).reshape(-1, 1)
    return (q.astype(np.float64) @ w.T) / s


# --------------------------------------------------------------------------- glue between two linears
def residual_add(x_bits: np.ndarray, r_bits: np.ndarray) -> np.ndarray:
    """model.py:330, :334: bf16 + bf16 -> bf16 (the fp32 sum rounded once more to bf16)."""
    return f32_to_bf16_bits(bf16_bits_to_f32(x_bits) + bf16_bits_to_f32(r_bits))


def relu2_mul(x13_bits: np.ndarray) -> np.ndarray:
    """model.py:243, :279-280: squared_relu(x1) * x3 on bf16 tensors, every op rounded to bf16."""
    f = x13_bits.shape[-1] // 2
    x1 = bf16_bits_to_f32(x13_bits[..., :f])
    x3 = bf16_bits_to_f32(x13_bits[..., f:])
    r = np.maximum(x1, np.float32(0))
    sq = bf16_bits_to_f32(f32_to_bf16_bits(r * r))
    return f32_to_bf16_bits(sq * x3)


def rmsnorm(h_bits: np.ndarray, w_bits: np.ndarray, eps: float) -> np.ndarray:
    """RMSNorm over the last axis, evaluated in float64 and rounded to bf16 (see the module header:
    parity unpinned, xformers is absent).  Returns bf16 storage."""
    h = bf16_bits_to_f32(h_bits).astype(np.float64)
    w = bf16_bits_to_f32(w_bits).astype(np.float64)
    y = h / np.sqrt((h * h).mean(axis=-1, keepdims=True) + float(eps)) * w
    return f32_to_bf16_bits(y.astype(np.float32))


def rope_rotate_half(x_bits: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """Rotary embedding of bf16 x [..., D] by angles given as cos / sin [..., D/2] (fp32): pair j is
    (x[j], x[j + D/2]).  Stands for xformers' rope_padded (model.py:218-229; absent dependency,
    parity unpinned).  fp32 arithmetic in the order x1*c - x2*s, x2*c + x1*s, one rounding to bf16."""
    x = bf16_bits_to_f32(x_bits)
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c, s = cos.astype(np.float32), sin.astype(np.float32)
    return f32_to_bf16_bits(np.concatenate([x1 * c - x2 * s, x2 * c + x1 * s], axis=-1).astype(np.float32))


def rope_adjacent(x_bits: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """As rope_rotate_half with pair j = (x[2j], x[2j + 1]): rope_padded's default pairing, the one the
    reference's checkpoints are laid out for (convert_TernaInfer.py:46-50 undoes the rotate-half row
    order of the source checkpoint).  Same arithmetic order and rounding; parity unpinned likewise."""
    x = bf16_bits_to_f32(x_bits)
    x1, x2 = x[..., 0::2], x[..., 1::2]
    c, s = cos.astype(np.float32), sin.astype(np.float32)
    out = np.empty_like(x)
    out[..., 0::2] = x1 * c - x2 * s
    out[..., 1::2] = x2 * c + x1 * s
    return f32_to_bf16_bits(out.astype(np.float32))


def attention_one_token(q_bits: np.ndarray, k_bits: np.ndarray, v_bits: np.ndarray, n: int, scale: float) -> np.ndarray:
    """softmax(scale * q K^T) V in float64 for one query per (sequence, head): q [B, H, D],
    k / v [B, KV, S, D], keys 0 .. n-1 valid, head h reads kv head h // (H // KV).  Stands for
    fmha.memory_efficient_attention_forward on the padded cache (model.py:231-233; absent
    dependency, parity unpinned).  Returns float64 [B, H, D]."""
    q = bf16_bits_to_f32(q_bits).astype(np.float64)
    k = bf16_bits_to_f32(k_bits).astype(np.float64)[:, :, :n]
    v = bf16_bits_to_f32(v_bits).astype(np.float64)[:, :, :n]
    rep = q.shape[1] // k.shape[1]
    k, v = np.repeat(k, rep, axis=1), np.repeat(v, rep, axis=1)
    sc = np.einsum("bhd,bhsd->bhs", q, k) * scale
    p = np.exp(sc - sc.max(axis=-1, keepdims=True))
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("bhs,bhsd->bhd", p, v)


def attention_new_tokens(q_bits: np.ndarray, k_bits: np.ndarray, v_bits: np.ndarray, pos: np.ndarray, scale: float) -> np.ndarray:
    """The same attention for T new tokens per sequence: q [B, H, T, D], k / v [B, KV, S, D] with the new tokens'
    rows already in their slots, token t sees the slots 0 .. pos[t] (model.py:231-233 with the causal bias of the
    prompt pass, generate.py:108-113; absent dependency, parity unpinned).  Each (t) row is attention_one_token
    over its own prefix -- evaluated that way, so the closed-form checks of attention_one_token carry over.
    Returns float64 [B, T, H, D]."""
    b, h, t, d = q_bits.shape
    out = np.empty((b, t, h, d), dtype=np.float64)
    for ti in range(t):
        out[:, ti] = attention_one_token(np.ascontiguousarray(q_bits[:, :, ti]), k_bits, v_bits, int(pos[ti]) + 1, scale)
    return out


def quant_weight_int8(w: np.ndarray):
    """convert_TernaInfer.py:159-163: ternarise by 1/mean(|W|); returns (int8 W, fp32 scale=1/s)."""
    w = np.asarray(w, dtype=np.float32)
    s = np.float32(1.0) / np.maximum(np.abs(w).mean(dtype=np.float32), np.float32(1e-5))
    t = np.clip(np.rint(w * s), -1, 1).astype(np.int8)
    return t, np.float32(1.0) / s


def algorithmic_bytes(n: int, k: int, n_sign_words: int, m: int, act_bytes: int, scale_bytes: int) -> int:
    """Bytes one call must move, counted on the reference-format tensors."""
    return (8 * (n * k // 64) + 4 * n_sign_words + 4 * (n * k // 4096 + 1) + 2 * (3 * n * k // 4096)
            + act_bytes * m * k + scale_bytes + 2 * m * n)


# --------------------------------------------------------------------------- C oracle binding
def build_c_oracle(force: bool = False) -> str:
    src = os.path.join(_HERE, "terna_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-s"])
    return _SO


class COracle:
    """ctypes face of terna_oracle.c."""

    def __init__(self):
        self.lib = ctypes.CDLL(build_c_oracle())
        L = self.lib
        vp, ci = ctypes.c_void_p, ctypes.c_int
        L.oracle_reorder.argtypes = [vp, vp, ci, ci]
        L.oracle_compress.argtypes = [vp, ci, ci, vp, vp, vp, vp]
        L.oracle_compress.restype = ctypes.c_long
        L.oracle_decode.argtypes = [vp, vp, vp, vp, ci, ci, vp]
        L.oracle_decode.restype = ci
        L.oracle_consumer_sim.argtypes = [vp, vp, vp, vp, ctypes.c_long, ci, vp]
        L.oracle_spmm_i8.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
        L.oracle_spmm_bf16.argtypes = [vp, vp, vp, ci, ci, ci, ci, vp]
        L.oracle_quant_input.argtypes = [vp, ci, ci, vp, vp]
        L.oracle_quant_input_mode.argtypes = [vp, ci, ci, ci, vp, vp]
        L.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16

    @staticmethod
    def _p(a):
        return a.ctypes.data_as(ctypes.c_void_p)

    def reorder(self, w):
        w = np.ascontiguousarray(w, dtype=np.int8)
        out = np.empty_like(w)
        self.lib.oracle_reorder(self._p(w), self._p(out), w.shape[0], w.shape[1])
        return out

    def encode(self, w):
        """ORIGINAL ternary matrix -> reference tuple order (vals, tile_off, median, bitmap)."""
        n, k = w.shape
        a = self.reorder(w)
        bitmap = np.zeros(n * k // 64, dtype=np.uint64)
        tile_off = np.zeros(n * k // 4096 + 1, dtype=np.int32)
        median = np.zeros(3 * n * k // 4096, dtype=np.uint16)
        words = np.zeros(n * k // 32 + 1, dtype=np.uint32)
        nw = self.lib.oracle_compress(self._p(a), n, k, self._p(bitmap), self._p(tile_off),
                                      self._p(median), self._p(words))
        assert nw >= 0
        return words[:nw].copy(), tile_off, median, bitmap

    def decode(self, words, tile_off, median, bitmap, n, k):
        words = np.ascontiguousarray(words, dtype=np.uint32)
        if words.size == 0:
            words = np.zeros(1, dtype=np.uint32)
        out = np.empty((n, k), dtype=np.int8)
        rc = self.lib.oracle_decode(self._p(np.ascontiguousarray(bitmap)), self._p(np.ascontiguousarray(tile_off)),
                                    self._p(np.ascontiguousarray(median)), self._p(words), n, k, self._p(out))
        if rc != 0:
            raise ValueError(f"oracle_decode: inconsistent stream (code {rc})")
        return out

    def consumer_sim(self, words, tile_off, median, bitmap, tile, band):
        words = np.ascontiguousarray(words, dtype=np.uint32)
        if words.size == 0:
            words = np.zeros(1, dtype=np.uint32)
        median = np.ascontiguousarray(median)
        out = np.empty((16, 64), dtype=np.int8)
        self.lib.oracle_consumer_sim(self._p(np.ascontiguousarray(bitmap)), self._p(np.ascontiguousarray(tile_off)),
                                     self._p(median), self._p(words), tile, band, self._p(out))
        return out

    def spmm_i8(self, x_q, w, s_bits, ws_bits, ws_num, mode):
        m, k = x_q.shape
        n = w.shape[0]
        out = np.empty((m, n), dtype=np.uint16)
        self.lib.oracle_spmm_i8(self._p(np.ascontiguousarray(x_q, dtype=np.int8)),
                                self._p(np.ascontiguousarray(w, dtype=np.int8)),
                                self._p(np.ascontiguousarray(s_bits, dtype=np.uint16)),
                                self._p(np.ascontiguousarray(ws_bits, dtype=np.uint16)),
                                ws_num, m, n, k, mode, self._p(out))
        return out

    def spmm_bf16(self, x_bits, w, scale, ws_num):
        m, k = x_bits.shape
        n = w.shape[0]
        out = np.empty((m, n), dtype=np.float64)
        self.lib.oracle_spmm_bf16(self._p(np.ascontiguousarray(x_bits, dtype=np.uint16)),
                                  self._p(np.ascontiguousarray(w, dtype=np.int8)),
                                  self._p(np.ascontiguousarray(scale, dtype=np.float32)),
                                  ws_num, m, n, k, self._p(out))
        return out

    def quant_input(self, x_bits, mode: int = QUANT_ROUNDED):
        m, k = x_bits.shape
        xq = np.empty((m, k), dtype=np.int8)
        s = np.empty(m, dtype=np.uint16)
        self.lib.oracle_quant_input_mode(self._p(np.ascontiguousarray(x_bits, dtype=np.uint16)), m, k, mode,
                                         self._p(xq), self._p(s))
        return xq, s
