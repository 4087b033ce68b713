"""Producer of the compressed ternary weight format -- host side of the C-ABI encoder.

Mirrors the interface of the reference's ``convert/convert_utils.py``: ``reorder_weight``
(:9-49) and ``compress_weight`` (:52-228, same argument, same 4-tuple in the same order
with the same dtypes), plus the ternarisation of ``convert/convert_TernaInfer.py:159-194``.
The work is done by ``ternaspmm_encode_i8`` in libternaspmm.so (C++, seconds for a 2B model
instead of the reference's Python loops).
"""
from __future__ import annotations

import ctypes
from typing import Tuple

import numpy as np
import torch

from . import _lib


def _np_ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def reorder_weight(weight: torch.Tensor) -> torch.Tensor:
    """16x16 block permutation of an int8 [N, K] matrix (convert_utils.py:9-49)."""
    assert weight.dtype == torch.int8
    n, k = weight.shape
    assert n % 16 == 0 and k % 16 == 0, "Must be a multiple of 16"
    # the library's permutation works on 16-bit storage; int8 values widen losslessly
    src = np.ascontiguousarray(weight.cpu().numpy().astype(np.int16)).view(np.uint16)
    dst = np.empty_like(src)
    _lib.load().reorder_WT_h(_np_ptr(src), _np_ptr(dst), n, k)
    return torch.from_numpy(dst.view(np.int16).astype(np.int8))


def compress_weight(weight: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Encode a ternary int8 [N, K] matrix (NOT yet reordered), as convert_utils.py:52 does.

    Returns ``(compressed_val uint32, TileOffsets_global int32, TileOffsets_median uint16,
    bitmap uint64)`` -- 1-D CPU tensors.
    """
    assert weight.dtype == torch.int8 and weight.dim() == 2
    lib = _lib.load()
    n, k = weight.shape
    sizes = (ctypes.c_int64 * 4)()
    rc = lib.ternaspmm_encode_sizes(n, k, *[ctypes.byref(sizes, 8 * j) for j in range(4)])
    if rc != 0:
        raise ValueError(f"compress_weight: N and K must be multiples of 64, got {n}x{k}")
    w = np.ascontiguousarray(weight.cpu().numpy())
    bitmap = np.empty(sizes[0], dtype=np.uint64)
    tile_off = np.empty(sizes[1], dtype=np.int32)
    median = np.empty(sizes[2], dtype=np.uint16)
    words = np.empty(max(int(sizes[3]), 1), dtype=np.uint32)
    nw = lib.ternaspmm_encode_i8(_np_ptr(w), n, k, _np_ptr(bitmap), _np_ptr(tile_off), _np_ptr(median),
                                 _np_ptr(words))
    if nw < 0:
        raise ValueError("compress_weight: weight has values outside {-1, 0, 1}")
    return (torch.from_numpy(words[:nw].copy()), torch.from_numpy(tile_off), torch.from_numpy(median),
            torch.from_numpy(bitmap))


def quant_weight_int8(weight: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Ternarise by 1/mean(|W|) (convert_TernaInfer.py:159-163) -> (int8 W, bf16 scale[1])."""
    s = 1.0 / weight.abs().mean().clamp_(min=1e-5)
    new_weight = (weight * s).round().clamp(-1, 1).to(torch.int8)
    new_scale = (1.0 / s).to(torch.bfloat16)
    return new_weight, new_scale.reshape(1)


def pack_weight_scale(scales) -> torch.Tensor:
    """Zero-pad per-sub-matrix scales to the 4-slot ``weight_scale`` (convert_TernaInfer.py:176-194)."""
    out = torch.zeros(4, dtype=torch.bfloat16)
    for j, s in enumerate(scales):
        out[j] = s
    return out
