"""Call site of the TernaSpMM path: the host-side mirror of the reference's ``model.py:21-153``.

``TernaInfer_linear`` / ``SpBitLinear`` / ``BF16BitLinear`` / ``get_global_workspace`` keep the
reference's names, arguments and behaviour (row padding to ``max(8, next_pow2(M))``,
``SPLIT_K = 7``, raw device pointers and the current stream handed to the C ABI).
``TernaInfer_linear_bf16`` / ``SpBitLinearBF16`` are the same call site for the
bf16-activation entry points this build adds.  PyTorch is only the owner of device memory
and streams here; all arithmetic happens in libternaspmm.so.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch
from torch import nn
from torch.nn import functional as F

from . import _lib

MAX_MATRIX_ELEMENTS = 13824 * 2560          # ModelArgs.max_matrix_elements, model.py:34

_GLOBAL_WORKSPACE = None


def get_global_workspace(device="cuda"):
    """One int8 scratch buffer shared by every layer (model.py:37-42).  The small-M kernels never
    touch it; a large-M call on the reference format transcodes the weight into its first N*K/4
    bytes (the 2-bit layout the MFMA kernel reads) instead of the reference's dense N*K copy."""
    global _GLOBAL_WORKSPACE
    if _GLOBAL_WORKSPACE is None:
        _GLOBAL_WORKSPACE = torch.empty(MAX_MATRIX_ELEMENTS, dtype=torch.int8, device=device)
    return _GLOBAL_WORKSPACE


def _p(t: torch.Tensor):
    return ctypes.c_void_p(t.data_ptr())


def TernaInfer_linear(input, compressed_val, TileOffsets_global, TileOffsets_median, bitmap,
                      workspace, s, ws, ws_num, out_features):
    """int8 activations x compressed ternary weight -> bf16 (model.py:45-92)."""
    lib = _lib.load()
    out_shape = list(input.shape)
    out_shape[-1] = out_features
    stream = torch.cuda.current_stream()

    M = input.shape[0]
    if len(out_shape) == 3:
        M *= input.shape[1]
    N = out_features
    K = input.shape[-1]
    SPLIT_K = 7

    M_padded = max(8, 1 << (M - 1).bit_length())
    pad_rows = M_padded - M
    if pad_rows > 0:
        input_padded = torch.cat([
            input.reshape(M, K),
            torch.empty((pad_rows, K), dtype=input.dtype, device=input.device)], dim=0)
        # the reference also reads s for the padding rows; give those reads memory to land in
        s_padded = torch.cat([s.reshape(M), torch.ones(pad_rows, dtype=s.dtype, device=s.device)])
    else:
        input_padded = input.reshape(M, K).contiguous()
        s_padded = s.reshape(M).contiguous()

    ret_padded = torch.empty((M_padded, N), dtype=torch.bfloat16, device=input.device)
    lib.bitlinear_TernaSpMM(
        _p(input_padded), _p(bitmap), _p(TileOffsets_global), _p(TileOffsets_median), _p(compressed_val),
        _p(ret_padded), _p(s_padded), _p(ws), ws_num, M_padded, N, K, SPLIT_K, _p(workspace),
        ctypes.c_void_p(stream.cuda_stream))
    return ret_padded[:M, :].reshape(*out_shape)


def TernaInfer_linear_bf16(input, compressed_val, TileOffsets_global, TileOffsets_median, bitmap,
                           scale, ws_num, out_features, route: str = "auto"):
    """bf16 activations x compressed ternary weight -> bf16, fp32 accumulate, fp32 scale[ws_num].
    No row padding: the entry point takes the true M."""
    lib = _lib.load()
    fn = {"auto": lib.bitlinear_TernaSpMM_bf16, "decode": lib.bitlinear_TernaSpMM_bf16_decode,
          "prefill": lib.bitlinear_TernaSpMM_bf16_prefill}[route]
    out_shape = list(input.shape)
    out_shape[-1] = out_features
    K = input.shape[-1]
    x = input.reshape(-1, K).contiguous()
    M = x.shape[0]
    assert x.dtype == torch.bfloat16 and scale.dtype == torch.float32
    out = torch.empty((M, out_features), dtype=torch.bfloat16, device=input.device)
    stream = torch.cuda.current_stream()
    fn(_p(x), _p(bitmap), _p(TileOffsets_global), _p(TileOffsets_median), _p(compressed_val), _p(out),
       _p(scale), ws_num, M, out_features, K, 1, None, ctypes.c_void_p(stream.cuda_stream))
    return out.reshape(*out_shape)


def repack_weight(compressed_val, TileOffsets_global, TileOffsets_median, bitmap, out_features, in_features):
    """Load-time repack of one matrix from the reference format to the library's P2 device layout
    (2 bits per weight, bit-exact; one kernel launch).  Returns an int8 device tensor of N*K/4 bytes."""
    lib = _lib.load()
    nbytes = lib.ternaspmm_packed_bytes(out_features, in_features)
    if nbytes < 0:
        raise ValueError(f"repack_weight: N and K must be multiples of 64, got {out_features}x{in_features}")
    packed = torch.empty(nbytes, dtype=torch.int8, device=bitmap.device)
    stream = torch.cuda.current_stream()
    lib.ternaspmm_repack(_p(bitmap), _p(TileOffsets_global), _p(TileOffsets_median), _p(compressed_val), _p(packed),
                         out_features, in_features, ctypes.c_void_p(stream.cuda_stream))
    return packed


def _check_rows(who, x, k=None, **others):
    """The kernels take pointers and sizes on trust: a tensor with the wrong number of elements would be read or written
    past its end on the GPU.  Raise here instead."""
    if x.dim() != 2 or (k is not None and x.shape[1] != k):
        raise ValueError(f"{who}: expected a [M, {k if k is not None else 'K'}] tensor, got {tuple(x.shape)}")
    for name, (t, numel) in others.items():
        if t is not None and t.numel() != numel:
            raise ValueError(f"{who}: {name} has {t.numel()} elements, expected {numel}")


def TernaInfer_linear_packed(input, packed, s, ws, ws_num, out_features):
    """int8 activations x P2-layout ternary weight -> bf16; the reference's epilogue rule by M
    (decode arithmetic for M <= 64, prefill arithmetic above).  No row padding needed."""
    lib = _lib.load()
    out_shape = list(input.shape)
    out_shape[-1] = out_features
    K = input.shape[-1]
    x = input.reshape(-1, K).contiguous()
    M = x.shape[0]
    _check_rows("TernaInfer_linear_packed", x, s=(s, M))
    if packed.numel() * packed.element_size() < out_features * K // 4 or ws.numel() < ws_num:
        raise ValueError("TernaInfer_linear_packed: packed weight or weight scales too small for this shape")
    out = torch.empty((M, out_features), dtype=torch.bfloat16, device=input.device)
    stream = torch.cuda.current_stream()
    work = get_global_workspace(input.device) if M > 64 else None      # large M: room for split-K partial sums
    lib.bitlinear_TernaSpMM_packed_ws(_p(x), _p(packed), _p(out), _p(s.reshape(M).contiguous()), _p(ws), ws_num,
                                      M, out_features, K, 0, _p(work) if work is not None else None,
                                      work.numel() if work is not None else 0, ctypes.c_void_p(stream.cuda_stream))
    return out.reshape(*out_shape)


def rmsnorm_quant(x, weight, eps, residual=None, quant=True):
    """Fused [residual add] -> RMSNorm -> [SpBitLinear.quant_input] in one launch
    (model.py:330/334 + the norm + model.py:120-123).  x, residual: bf16 [M, K]; weight: bf16 [K].
    Returns (xq int8 [M, K], s bf16 [M], h) when quant else (y bf16 [M, K], h); h is the bf16 sum
    x + residual (x itself when residual is None)."""
    m, k = x.shape
    _check_rows("rmsnorm_quant", x, residual=(residual, m * k), weight=(weight, k))
    x = x.contiguous()
    lib = _lib.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    h = x
    if residual is not None:
        residual = residual.contiguous()
        h = torch.empty_like(x)
    if quant:
        xq = torch.empty((m, k), dtype=torch.int8, device=x.device)
        s = torch.empty(m, dtype=torch.bfloat16, device=x.device)
        lib.ternaspmm_rmsnorm_quant(_p(x), _p(residual) if residual is not None else None,
                                    _p(h) if residual is not None else None, _p(weight), float(eps), None, _p(xq),
                                    _p(s), m, k, stream)
        return xq, s, h
    y = torch.empty_like(x)
    lib.ternaspmm_rmsnorm_quant(_p(x), _p(residual) if residual is not None else None,
                                _p(h) if residual is not None else None, _p(weight), float(eps), _p(y), None, None,
                                m, k, stream)
    return y, h


def rmsnorm_linear_packed(x, norm_weight, eps, packed, ws, ws_num, out_features, residual=None):
    """[residual add] -> RMSNorm -> quant_input -> int8 TernaSpMM on a P2 weight.  One launch where that is
    faster and the library supports the shape -- every workgroup of the fused kernel repeats the prologue
    arithmetic, which pays at M = 1 (4.0-6.6 us against 6.6-8.8 us on MI355X), up to M = 4 with the 2- and 4-row
    variants and, without a residual, up to M = 8 (6.3 against 6.9 us; with one it is 7.7 against 7.2) -- else
    rmsnorm_quant + TernaInfer_linear_packed.
    x, residual: bf16 [M, K].  Returns (out bf16 [M, out_features], h = x + residual)."""
    m, k = x.shape
    _check_rows("rmsnorm_linear_packed", x, residual=(residual, m * k), norm_weight=(norm_weight, k))
    if packed.numel() * packed.element_size() < out_features * k // 4 or ws.numel() < ws_num:
        raise ValueError("rmsnorm_linear_packed: packed weight or weight scales too small for this shape")
    x = x.contiguous()
    lib = _lib.load()
    h = x
    if residual is not None:
        residual = residual.contiguous()
        h = torch.empty_like(x)
    out = torch.empty((m, out_features), dtype=torch.bfloat16, device=x.device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    one_launch = m <= 4 or (m <= 8 and residual is None)
    done = one_launch and lib.bitlinear_TernaSpMM_packed_fused(
        _p(x), _p(residual) if residual is not None else None, _p(h) if residual is not None else None,
        _p(norm_weight), float(eps), _p(packed), _p(out), _p(ws), ws_num, None, None, m, out_features, k, stream)
    if done:
        return out, h
    xq, s, h = rmsnorm_quant(x, norm_weight, eps, residual=residual)
    return TernaInfer_linear_packed(xq, packed, s, ws, ws_num, out_features), h


def attention_merge_rmsnorm_linear_packed(partial, splits, heads, head_dim, norm_weight, eps, packed, ws, ws_num, out_features,
                                          sequences=1):
    """The O projection of a decode step fed by the partial results of a split attention launch
    (ternaspmm_rope_decode_attention_partial over `sequences` sequences): for one sequence merge -> RMSNorm -> quant_input
    -> int8 TernaSpMM in one launch where the library supports the shape; for more, merge + norm + quantisation in one
    launch (ternaspmm_attention_merge_rmsnorm_quant) and the linear on its rows; else ternaspmm_attention_merge +
    rmsnorm_linear_packed.  partial: fp32 device buffer of ternaspmm_attention_partial_bytes(sequences, ...);
    returns out bf16 [sequences, out_features]."""
    lib = _lib.load()
    k = heads * head_dim
    need = lib.ternaspmm_attention_partial_bytes(sequences, heads, head_dim)
    if sequences < 1 or need < 0 or partial.numel() * partial.element_size() < need:
        raise ValueError(f"partial buffer of {partial.numel() * partial.element_size()} bytes does not hold {sequences} sequences")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if sequences == 1:
        out = torch.empty((1, out_features), dtype=torch.bfloat16, device=partial.device)
        if lib.bitlinear_TernaSpMM_packed_fused_attn(_p(partial), splits, head_dim, _p(norm_weight), float(eps), _p(packed), _p(out),
                                                     _p(ws), ws_num, None, None, 1, out_features, k, stream):
            return out
    else:
        # several sequences: merge + norm + quantisation once per sequence in one launch, then the linear on the quantised rows
        mq = attention_merge_rmsnorm_quant(partial, splits, heads, head_dim, norm_weight, eps, sequences)
        if mq is not None:
            return TernaInfer_linear_packed(mq[0], packed, mq[1], ws, ws_num, out_features)
    o = torch.empty((sequences, k), dtype=torch.bfloat16, device=partial.device)
    lib.ternaspmm_attention_merge(_p(partial), splits, _p(o), sequences, heads, head_dim, stream)
    return rmsnorm_linear_packed(o, norm_weight, eps, packed, ws, ws_num, out_features)[0]


def attention_merge_rmsnorm_quant(partial, splits, heads, head_dim, norm_weight, eps, sequences, want_output=False):
    """ternaspmm_attention_merge + rmsnorm_quant in one launch (one workgroup per sequence): the quantised input of the O
    projection from the partial results of a split attention launch.  Returns (xq int8 [sequences, heads * head_dim],
    s bf16 [sequences], o) -- o the merged attention output with `want_output`, else None -- or None where the library
    does not take the shape (nothing enqueued)."""
    lib = _lib.load()
    k = heads * head_dim
    need = lib.ternaspmm_attention_partial_bytes(sequences, heads, head_dim)
    if sequences < 1 or need < 0 or partial.numel() * partial.element_size() < need:
        raise ValueError(f"partial buffer of {partial.numel() * partial.element_size()} bytes does not hold {sequences} sequences")
    if norm_weight.numel() != k or norm_weight.dtype != torch.bfloat16:
        raise ValueError("attention_merge_rmsnorm_quant: the norm weight is a bf16 vector of heads * head_dim elements")
    dev = partial.device
    xq = torch.empty((sequences, k), dtype=torch.int8, device=dev)
    s = torch.empty(sequences, dtype=torch.bfloat16, device=dev)
    o = torch.empty((sequences, k), dtype=torch.bfloat16, device=dev) if want_output else None
    rc = lib.ternaspmm_attention_merge_rmsnorm_quant(_p(partial), splits, _p(norm_weight), float(eps), _p(o) if o is not None else None, _p(xq), _p(s), sequences, heads,
                                                     head_dim, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return None if rc != 0 else (xq, s, o)


def relu2_mul_rmsnorm_linear_packed(x13, norm_weight, eps, packed, ws, ws_num, out_features):
    """squared_relu(x1) * x3 -> RMSNorm -> quant_input -> int8 TernaSpMM on a P2 weight: one launch for up to four
    rows where the library supports the shape, else relu2_mul_rmsnorm_quant + TernaInfer_linear_packed.
    x13: bf16 [M, 2F].  Returns out bf16 [M, out_features]."""
    m, f2 = x13.shape
    _check_rows("relu2_mul_rmsnorm_linear_packed", x13, norm_weight=(norm_weight, f2 // 2))
    if f2 % 2 or packed.numel() * packed.element_size() < out_features * (f2 // 2) // 4 or ws.numel() < ws_num:
        raise ValueError("relu2_mul_rmsnorm_linear_packed: packed weight or weight scales too small for this shape")
    x13 = x13.contiguous()
    lib = _lib.load()
    out = torch.empty((m, out_features), dtype=torch.bfloat16, device=x13.device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if m <= 4 and lib.bitlinear_TernaSpMM_packed_fused_glu(_p(x13), _p(norm_weight), float(eps), _p(packed), _p(out), _p(ws),
                                                         ws_num, None, None, m, out_features, f2 // 2, stream):
        return out
    xq, s = relu2_mul_rmsnorm_quant(x13, norm_weight, eps)
    return TernaInfer_linear_packed(xq, packed, s, ws, ws_num, out_features)


def relu2_mul_rmsnorm_quant(x13, weight, eps, quant=True):
    """Fused squared_relu(x1) * x3 -> ffn_sub_norm -> [quant_input] (model.py:279-281 + 120-123).
    x13: bf16 [M, 2F].  Returns (xq int8 [M, F], s bf16 [M]) when quant else y bf16 [M, F]."""
    m, f2 = x13.shape
    f = f2 // 2
    _check_rows("relu2_mul_rmsnorm_quant", x13, weight=(weight, f))
    x13 = x13.contiguous()
    lib = _lib.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if quant:
        xq = torch.empty((m, f), dtype=torch.int8, device=x13.device)
        s = torch.empty(m, dtype=torch.bfloat16, device=x13.device)
        lib.ternaspmm_relu2_mul_rmsnorm_quant(_p(x13), _p(weight), float(eps), None, _p(xq), _p(s), m, f, stream)
        return xq, s
    y = torch.empty((m, f), dtype=torch.bfloat16, device=x13.device)
    lib.ternaspmm_relu2_mul_rmsnorm_quant(_p(x13), _p(weight), float(eps), _p(y), None, None, m, f, stream)
    return y


class FusedLinearDesc(ctypes.Structure):
    """ternaspmm_fused_linear_desc of include/ternaspmm.h."""
    _fields_ = [(n, ctypes.c_int) for n in ("prologue", "epilogue", "M", "N", "K", "ws_num")] + [("eps", ctypes.c_float)] + \
               [(n, ctypes.c_int) for n in ("stats_count", "attention_splits", "head_dim")] + \
               [(n, ctypes.c_void_p) for n in ("x", "stats_in", "norm_weight", "packed", "ws", "out", "residual",
                                               "next_norm_weight", "stats_out", "raw_out", "xq_out", "s_out", "s_in")]


PROLOGUE_NORM, PROLOGUE_ATTENTION, PROLOGUE_STATS, PROLOGUE_QUANTISED = 0, 1, 2, 3
EPILOGUE_STORE, EPILOGUE_RESIDUAL, EPILOGUE_GATE = 0, 1, 2


def row_stats(h, norm_weight):
    """Partials of the norm statistics of h bf16 [M, K] under `norm_weight` (ternaspmm_row_stats): fp32 [M, count, 2]."""
    m, k = h.shape
    _check_rows("row_stats", h, norm_weight=(norm_weight, k))
    lib = _lib.load()
    count = lib.ternaspmm_row_stats_count(k)
    if count < 1:
        raise ValueError(f"row_stats: unsupported K={k}")
    out = torch.empty((m, count, 2), dtype=torch.float32, device=h.device)
    lib.ternaspmm_row_stats(_p(h.contiguous()), _p(norm_weight), _p(out), m, k, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return out


def step_inputs(tokens, pos, embedding, rope_table, norm_weight):
    """The inputs of a single-token step in one launch (ternaspmm_step_inputs): tokens int64 [B] (any shape with B
    elements), pos int64 [1] (one position for all) or [B], embedding bf16 [V, K], rope_table fp32 [S, 2, half].
    Returns (x bf16 [B, K], partials fp32 [B, count, 2] under `norm_weight`, cos fp32 [B, half], sin fp32 [B, half])."""
    b = tokens.numel()
    v, k = embedding.shape
    s_len, two, half = rope_table.shape
    tokens, pos = tokens.reshape(-1).contiguous(), pos.reshape(-1).contiguous()      # (copies only where a caller passed a strided view)
    if tokens.dtype != torch.int64 or pos.dtype != torch.int64 or pos.numel() not in (1, b) or two != 2 or rope_table.dtype != torch.float32 \
            or embedding.dtype != torch.bfloat16 or not (embedding.is_contiguous() and rope_table.is_contiguous()):
        raise ValueError("step_inputs: tokens / pos int64, embedding bf16 [V, K] and rope_table fp32 [S, 2, half] contiguous")
    _check_rows("step_inputs", embedding, norm_weight=(norm_weight, k))
    lib = _lib.load()
    count = lib.ternaspmm_row_stats_count(k)
    if count < 1:
        raise ValueError(f"step_inputs: unsupported K={k}")
    x = torch.empty((b, k), dtype=torch.bfloat16, device=embedding.device)
    stats = torch.empty((b, count, 2), dtype=torch.float32, device=embedding.device)
    rope = torch.empty((2, b, half), dtype=torch.float32, device=embedding.device)
    got = lib.ternaspmm_step_inputs(_p(tokens), _p(pos), int(pos.numel() == b and b > 1), _p(embedding), v, k, _p(rope_table), s_len, half,
                                    _p(norm_weight), _p(x), _p(stats), _p(rope), b, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    if got != count:
        raise ValueError(f"step_inputs: the library refused the launch (B={b} V={v} K={k} S={s_len} half={half})")
    return x, stats, rope[0], rope[1]


def quant_from_stats(h, stats, norm_weight, eps):
    """Norm + quant_input of h bf16 [M, K] from the partials its producer left (ternaspmm_quant_from_stats):
    (xq int8 [M, K], s bf16 [M])."""
    m, k = h.shape
    _check_rows("quant_from_stats", h, norm_weight=(norm_weight, k))
    if stats.dtype != torch.float32 or stats.dim() != 3 or stats.shape[0] != m or stats.shape[2] != 2 or not stats.is_contiguous():
        raise ValueError("quant_from_stats: stats must be a contiguous fp32 [M, count, 2] tensor")
    xq = torch.empty((m, k), dtype=torch.int8, device=h.device)
    s = torch.empty(m, dtype=torch.bfloat16, device=h.device)
    if _lib.load().ternaspmm_quant_from_stats(_p(h.contiguous()), _p(stats), stats.shape[1], _p(norm_weight), float(eps), _p(xq), _p(s),
                                             m, k, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) != 0:
        raise ValueError(f"quant_from_stats: unsupported shape M={m} K={k}")
    return xq, s


def interleave_gate_up(packed, out_features, in_features):
    """Load time: the band order TERNASPMM_EPILOGUE_GATE reads (ternaspmm_interleave_gate_up) of a P2 gate+up matrix."""
    out = torch.empty_like(packed)
    if _lib.load().ternaspmm_interleave_gate_up(_p(packed), _p(out), out_features, in_features,
                                               ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) != 0:
        raise ValueError(f"interleave_gate_up: unsupported shape {out_features}x{in_features}")
    return out


def fused_linear(x, norm_weight, eps, packed, ws, ws_num, out_features, in_features, *, stats=None, attention=None, quantised=None,
                 epilogue=EPILOGUE_STORE, residual=None, next_norm_weight=None, want_raw=False, publish=False):
    """One launch of ternaspmm_fused_linear (include/ternaspmm.h): prologue -> ternary matmul on a P2 weight -> epilogue.
    x: h bf16 [M, K], with `stats` (fp32 [M, count, 2]) when its producer left the norm statistics; or, with
    `attention` = (splits, head_dim), the fp32 partial results of a split attention launch (one sequence); or, with
    `quantised` = s (bf16 [M]), int8 activations that are quantised already (norm_weight is then not used).
    Returns (out, stats_out, raw, xq, s) -- stats_out for the producing epilogues, raw with `want_raw`, (xq, s) with
    `publish`, None otherwise -- or None when the library does not support the combination (nothing was enqueued)."""
    lib = _lib.load()
    k, n = in_features, out_features
    if attention is not None:
        m, pro = 1, PROLOGUE_ATTENTION
    elif quantised is not None:
        m, pro = x.shape[0], PROLOGUE_QUANTISED
        _check_rows("fused_linear", x, k, s=(quantised, m))
        if x.dtype != torch.int8 or quantised.dtype != torch.bfloat16:
            raise ValueError("fused_linear: quantised activations are int8 with bf16 scales")
        x = x.contiguous()
    else:
        m = x.shape[0]
        _check_rows("fused_linear", x, k, norm_weight=(norm_weight, k))
        x = x.contiguous()
        pro = PROLOGUE_STATS if stats is not None else PROLOGUE_NORM
    if packed.numel() * packed.element_size() < n * k // 4 or ws.numel() < ws_num:
        raise ValueError("fused_linear: packed weight or weight scales too small for this shape")
    dev = packed.device
    out_cols = n // 2 if epilogue == EPILOGUE_GATE else n
    d = FusedLinearDesc()
    d.prologue, d.epilogue, d.M, d.N, d.K, d.ws_num, d.eps = pro, epilogue, m, n, k, ws_num, float(eps)
    d.x, d.packed, d.ws = x.data_ptr(), packed.data_ptr(), ws.data_ptr()
    d.norm_weight = norm_weight.data_ptr() if norm_weight is not None else None
    if quantised is not None:
        quantised = quantised.contiguous()
        d.s_in = quantised.data_ptr()
    if stats is not None:
        if stats.dtype != torch.float32 or stats.dim() != 3 or stats.shape[0] != m or stats.shape[2] != 2 or not stats.is_contiguous():
            raise ValueError("fused_linear: stats must be a contiguous fp32 [M, count, 2] tensor")
        d.stats_in, d.stats_count = stats.data_ptr(), stats.shape[1]
    if attention is not None:
        d.attention_splits, d.head_dim = attention
    out = torch.empty((m, out_cols), dtype=torch.bfloat16, device=dev)
    d.out = out.data_ptr()
    stats_out = raw = xq = s = None
    if epilogue != EPILOGUE_STORE:
        if next_norm_weight is None or next_norm_weight.numel() != out_cols:
            raise ValueError("fused_linear: a producing epilogue needs the next norm's weights")
        stats_out = torch.empty((m, out_cols // 16, 2), dtype=torch.float32, device=dev)
        d.next_norm_weight, d.stats_out = next_norm_weight.data_ptr(), stats_out.data_ptr()
    if epilogue == EPILOGUE_RESIDUAL:
        if residual is None or residual.numel() != m * n or residual.dtype != torch.bfloat16:
            raise ValueError("fused_linear: the residual epilogue needs a bf16 [M, N] stream")
        residual = residual.contiguous()
        d.residual = residual.data_ptr()
        if want_raw:
            raw = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
            d.raw_out = raw.data_ptr()
    if publish:
        xq = torch.empty((m, k), dtype=torch.int8, device=dev)
        s = torch.empty(m, dtype=torch.bfloat16, device=dev)
        d.xq_out, d.s_out = xq.data_ptr(), s.data_ptr()
    rc = lib.ternaspmm_fused_linear(ctypes.byref(d), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    if rc < 0:
        return None
    return out, stats_out, raw, xq, s


def lm_head(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Logits of a decode step: F.linear(x, weight) for bf16 x [M, K] with M <= 16 and the bf16 output
    (tied embedding) matrix weight [V, K] (model.py:367, 449-455), as one HBM-bound pass over the matrix."""
    assert x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.dim() == 2 and weight.dim() == 2
    assert x.is_contiguous() and weight.is_contiguous() and x.shape[1] == weight.shape[1]
    m, k = x.shape
    v = weight.shape[0]
    if m > 16 or k % 32 or m * (2 * k + 16) > 160 * 1024:
        raise ValueError(f"lm_head: unsupported shape M={m} K={k}")
    if out is None:
        out = torch.empty((m, v), dtype=torch.bfloat16, device=x.device)
    assert out.dtype == torch.bfloat16 and out.shape == (m, v) and out.is_contiguous()
    _lib.load().ternaspmm_lm_head_bf16(_p(x), _p(weight), _p(out), m, v, k, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return out


def argmax_rows(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Greedy sampling: index of the largest logit per row of a bf16 [B, V] tensor -> int64 [B, 1]
    (torch.argmax(logits, dim=-1), generate.py:283; ties to the lowest index).  `out`, if given, is
    an int64 tensor of B elements that receives the result in place."""
    assert logits.dtype == torch.bfloat16 and logits.dim() == 2 and logits.is_contiguous()
    b, v = logits.shape
    if out is None:
        out = torch.empty((b, 1), dtype=torch.int64, device=logits.device)
    assert out.dtype == torch.int64 and out.numel() == b and out.is_contiguous()
    _lib.load().ternaspmm_argmax_bf16(_p(logits), _p(out), b, v, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return out


def greedy_step_state(batch: int, device="cuda") -> torch.Tensor:
    """Zero-filled scratch of `greedy_step` for `batch` rows; allocate once, launches restore it."""
    return torch.zeros(_lib.load().ternaspmm_greedy_step_state_bytes(batch) // 8, dtype=torch.int64, device=device)


def greedy_step(logits: torch.Tensor, tok: torch.Tensor, history: Optional[torch.Tensor], counters: Optional[torch.Tensor],
                state: torch.Tensor) -> torch.Tensor:
    """One launch for the tail of a greedy decode step (generate.py:283-305): tok[b] = argmax(logits[b]);
    history[b, counters[1]] = tok[b] while there is room; counters += 1 (int64 [2]: next cache slot, tokens stored).
    `state` comes from `greedy_step_state`."""
    assert logits.dtype == torch.bfloat16 and logits.dim() == 2 and logits.is_contiguous()
    b, v = logits.shape
    assert tok.dtype == torch.int64 and tok.numel() == b and tok.is_contiguous()
    hist_len = 0
    if history is not None:
        assert history.dtype == torch.int64 and history.dim() == 2 and history.shape[0] == b and history.is_contiguous()
        hist_len = history.shape[1]
    if counters is not None:
        assert counters.dtype == torch.int64 and counters.numel() == 2 and counters.is_contiguous()
    assert state.dtype == torch.int64 and state.numel() * 8 >= _lib.load().ternaspmm_greedy_step_state_bytes(b)
    _lib.load().ternaspmm_greedy_step_bf16(_p(logits), _p(tok), _p(history) if history is not None else None, hist_len,
                                           _p(counters) if counters is not None else None, _p(state), b, v,
                                           ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return tok


QUANT_ROUNDED, QUANT_COMPILED, QUANT_EAGER = 0, 1, 2


def quant_input(input: torch.Tensor, mode: Optional[int] = None):
    """Per-row int8 quantisation of the activations (model.py:120-123): s = 127 / max(max|x|, 1e-5),
    x_q = clamp(round(x * s), -128, 127).  The reference's two lines leave the intermediate precision to PyTorch;
    `mode` (default: the library's current ternaspmm_quant_mode, which the prologue kernels follow too) says which
    evaluation is reproduced:
      QUANT_ROUNDED   fp32 arithmetic, s rounded to bf16, and that rounded s both multiplies here and divides in the
                      epilogue (the library's default);
      QUANT_COMPILED  the method as the reference ships it, under @torch.compile: fp32 arithmetic, the UNROUNDED
                      quotient multiplies, the returned s is its bf16 rounding;
      QUANT_EAGER     the same lines without torch.compile on a bf16 tensor: every op rounds to bf16.
    The three differ from each other on a few percent of the elements, by one step (two at most).
    Returns (x_q int8, s bf16 [..., 1])."""
    if mode is None:
        mode = _lib.load().ternaspmm_quant_mode(-1)
    if mode == QUANT_EAGER:                       # the reference's two lines as they stand, on the bf16 tensor
        x = input.to(torch.bfloat16)
        s = 127 / x.abs().max(dim=-1, keepdim=True).values.clamp_(min=1e-5)
        return (x * s).round().clamp(-128, 127).to(torch.int8), s
    x = input.float()
    amax = x.abs().amax(dim=-1, keepdim=True).clamp_(min=1e-5)
    if mode == QUANT_COMPILED:                    # `127 / t` is t.reciprocal() * 127; nothing is rounded to bf16 on the way
        t = amax.reciprocal() * 127.0
        return (x * t).round().clamp(-128, 127).to(torch.int8), t.to(torch.bfloat16)
    s = (127.0 / amax).to(torch.bfloat16)
    return (x * s.float()).round().clamp(-128, 127).to(torch.int8), s


class _CompressedWeight(nn.Module):
    """Holds the four format tensors + ``weight_scale`` under the reference's checkpoint keys
    (convert_TernaInfer.py:204-209, model.py:110-116)."""

    def __init__(self, in_features: int, out_features: int, dic: dict, key: str):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        dev = "cuda"
        mk = lambda t: torch.nn.Parameter(t.to(dev), requires_grad=False)
        self.weight_compressed_val = mk(dic[key + ".weight_compressed_val"])
        self.weight_TileOffsets_global = mk(dic[key + ".weight_TileOffsets_global"])
        self.weight_TileOffsets_median = mk(dic[key + ".weight_TileOffsets_median"])
        self.weight_bitmap = mk(dic[key + ".weight_bitmap"])
        ws = dic[key + ".weight_scale"]
        self.weight_scale = mk(ws)
        self.ws_num = len(ws[ws != 0])


class SpBitLinear(_CompressedWeight):
    """Ternary linear on int8-quantised activations (model.py:96-133).  With ``repack=True`` the
    weight is repacked once at construction and every call runs on the P2 layout."""

    def __init__(self, in_features: int, out_features: int, dic: dict, key: str, bias: bool = False,
                 repack: bool = False):
        super().__init__(in_features, out_features, dic, key)
        self.weight_packed = None
        if repack:
            self.weight_packed = torch.nn.Parameter(
                repack_weight(self.weight_compressed_val, self.weight_TileOffsets_global,
                              self.weight_TileOffsets_median, self.weight_bitmap, out_features, in_features),
                requires_grad=False)

    def quant_input(self, input):
        return quant_input(input)

    def forward(self, input):
        input, s = self.quant_input(input)
        if self.weight_packed is not None:
            return TernaInfer_linear_packed(input, self.weight_packed, s, self.weight_scale,
                                            self.ws_num, self.out_features)
        return TernaInfer_linear(
            input, self.weight_compressed_val, self.weight_TileOffsets_global, self.weight_TileOffsets_median,
            self.weight_bitmap, get_global_workspace(), s, self.weight_scale, self.ws_num, self.out_features)


class SpBitLinearBF16(_CompressedWeight):
    """Ternary linear on bf16 activations (no activation quantisation)."""

    def __init__(self, in_features: int, out_features: int, dic: dict, key: str):
        super().__init__(in_features, out_features, dic, key)
        self.scale_f32 = torch.nn.Parameter(self.weight_scale.float(), requires_grad=False)

    def forward(self, input):
        return TernaInfer_linear_bf16(
            input, self.weight_compressed_val, self.weight_TileOffsets_global, self.weight_TileOffsets_median,
            self.weight_bitmap, self.scale_f32, self.ws_num, self.out_features)


class BF16BitLinear(nn.Module):
    """Dense reference semantics (model.py:135-153): quantise activations, bf16 GEMM, divide by s."""

    def __init__(self, in_features: int, out_features: int, dic: dict, key: str):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight = torch.nn.Parameter(dic[key + ".weight"].cuda(), requires_grad=False)

    def quant_input(self, input):
        return quant_input(input)

    def forward(self, input):
        input, s = self.quant_input(input)
        return F.linear(input.to(torch.bfloat16), self.weight) / s
