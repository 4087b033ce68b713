"""Producer of the compressed ternary weight format -- host side of the C-ABI encoder.

Mirrors the interface of the reference's ``convert/convert_utils.py``: ``reorder_weight``
(:9-49) and ``compress_weight`` (:52-228, same argument, same 4-tuple in the same order
with the same dtypes), plus the ternarisation of ``convert/convert_TernaInfer.py:159-194``.
The work is done by ``ternaspmm_encode_i8`` in libternaspmm.so (C++, seconds for a 2B model
instead of the reference's Python loops).
"""
from __future__ import annotations

import ctypes
import os
from dataclasses import dataclass
from typing import Dict, Optional, Tuple

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


# --------------------------------------------------------------------------- whole checkpoints
# The reference's converter (convert/convert_TernaInfer.py) turns one bf16 state dict into three
# files; the functions below do the same on dictionaries, with the C++ encoder doing the
# compression, so that 2 G weights convert in seconds rather than hours.
CKPT_BF16 = "model_bf16.pt"                                          # convert_TernaInfer.py:244
CKPT_TERNARY = "model_TernaInfer_TernaryWeights.pt"                  # :267
CKPT_NON_TERNARY = "model_embeddings_and_norms_non_ternary.pt"       # :268


@dataclass
class CheckpointShape:
    """The dimensions the converter needs to split the fused matrices (convert_TernaInfer.py:99-109)."""
    dim: int = 2560
    n_heads: int = 20
    n_kv_heads: int = 5
    ffn_dim: int = 6912
    n_layers: int = 30

    @property
    def kv_dim(self) -> int:
        return self.dim // self.n_heads * self.n_kv_heads


def _pairs_to_adjacent(w: torch.Tensor, heads: int) -> torch.Tensor:
    """Rows of a q / k projection from the source checkpoint's order (per head: first halves of all
    rotary pairs, then second halves) to adjacent pairs, the order rope_padded expects
    (convert_TernaInfer.py:46-50: '(h l d) i -> (h d l) i', l = 2)."""
    rows, cols = w.shape
    d = rows // (heads * 2)
    return w.reshape(heads, 2, d, cols).transpose(1, 2).reshape(rows, cols)


def convert_back(safetensors_path: str, cfg: Optional[CheckpointShape] = None) -> Dict[str, torch.Tensor]:
    """Source checkpoint (`model.layers.N.self_attn.q_proj.weight`, ...) -> the state dict the model
    code names (`layers.N.attention.wqkv.weight`, ...), with q | k | v and gate | up fused along the
    rows and the q / k rows re-ordered for adjacent rotary pairs (convert_TernaInfer.py:52-95)."""
    from safetensors.torch import load_file
    cfg = cfg or CheckpointShape()
    src = load_file(safetensors_path)
    out: Dict[str, torch.Tensor] = {}
    for n in range(cfg.n_layers):
        a, f, dst = f"model.layers.{n}.self_attn.", f"model.layers.{n}.mlp.", f"layers.{n}."
        wq = _pairs_to_adjacent(src[a + "q_proj.weight"], cfg.n_heads)
        wk = _pairs_to_adjacent(src[a + "k_proj.weight"], cfg.n_kv_heads)
        out[dst + "attention.wqkv.weight"] = torch.cat([wq, wk, src[a + "v_proj.weight"]], dim=0)
        out[dst + "attention.wo.weight"] = src[a + "o_proj.weight"]
        out[dst + "attention_norm.weight"] = src[f"model.layers.{n}.input_layernorm.weight"]
        out[dst + "ffn_norm.weight"] = src[f"model.layers.{n}.post_attention_layernorm.weight"]
        out[dst + "attention.attn_sub_norm.weight"] = src[a + "attn_sub_norm.weight"]
        out[dst + "feed_forward.ffn_sub_norm.weight"] = src[f + "ffn_sub_norm.weight"]
        out[dst + "feed_forward.w13.weight"] = torch.cat([src[f + "gate_proj.weight"], src[f + "up_proj.weight"]], dim=0)
        out[dst + "feed_forward.w2.weight"] = src[f + "down_proj.weight"]
    out["tok_embeddings.weight"] = src["model.embed_tokens.weight"]
    out["output.weight"] = src["model.embed_tokens.weight"]
    out["norm.weight"] = src["model.norm.weight"]
    return out


def _sub_matrices(key: str, value: torch.Tensor, cfg: CheckpointShape):
    """Row blocks of a (possibly fused) linear weight that are ternarised with a scale of their own:
    wqkv -> q | k | v, w13 -> w1 | w3, wo / w2 -> the matrix; None for every other tensor
    (convert_TernaInfer.py:165-192)."""
    if "wqkv" in key:
        return [value[:cfg.dim], value[cfg.dim:cfg.dim + cfg.kv_dim], value[cfg.dim + cfg.kv_dim:]]
    if "w13" in key:
        return [value[:cfg.ffn_dim], value[cfg.ffn_dim:]]
    if "w2" in key or "wo" in key:
        return [value]
    return None


@torch.inference_mode()
def convert_bitnet_checkpoint_to_bf16(state: Dict[str, torch.Tensor], cfg: Optional[CheckpointShape] = None):
    """Dense reference weights: every sub-matrix replaced by round(W s).clamp(-1, 1) / s, s = 1/mean|W|
    (convert_TernaInfer.py:111-151)."""
    cfg = cfg or CheckpointShape()
    out = {}
    for key, value in state.items():
        parts = _sub_matrices(key, value, cfg)
        if parts is None:
            out[key] = value.clone()
            continue
        dense = []
        for w in parts:
            s = 1.0 / w.abs().mean().clamp_(min=1e-5)
            dense.append((w * s).round().clamp(-1, 1) / s)
        out[key] = torch.cat(dense, dim=0)
    return out


@torch.inference_mode()
def convert_bitnet_checkpoint_to_int8(state: Dict[str, torch.Tensor], cfg: Optional[CheckpointShape] = None):
    """Ternary int8 weights under their own keys plus `<...>.weight_scale` = bf16[4] (one scale per
    sub-matrix, zero padded); `output.weight` is dropped, everything else is passed through
    (convert_TernaInfer.py:154-199)."""
    cfg = cfg or CheckpointShape()
    out = {}
    for key, value in state.items():
        parts = _sub_matrices(key, value, cfg)
        if parts is None:
            if "output.weight" not in key:
                out[key] = value.clone()
            continue
        quantised = [quant_weight_int8(w) for w in parts]
        out[key] = torch.cat([w for w, _ in quantised], dim=0)
        out[key.replace("weight", "weight_scale")] = pack_weight_scale([sc[0] for _, sc in quantised])
    return out


def convert_one_weight(item):
    """(key, int8 matrix) -> the four format tensors under the reference's key suffixes
    (convert_TernaInfer.py:201-209)."""
    key, weight = item
    vals, off, med, bm = compress_weight(weight)
    return {key + "_compressed_val": vals, key + "_TileOffsets_global": off, key + "_TileOffsets_median": med,
            key + "_bitmap": bm}


def compress_checkpoint(int8_model: Dict[str, torch.Tensor], workers: Optional[int] = None):
    """Split an int8 checkpoint into (ternary_result, non_ternary) as convert_TernaInfer.py:249-268 does:
    every 2-D tensor of a layer is compressed, the rest (embedding, norms, weight scales) is kept.
    The encoder runs outside the interpreter lock, so a thread pool is enough."""
    from concurrent.futures import ThreadPoolExecutor
    tasks = [(k, v) for k, v in int8_model.items() if v.dim() == 2 and "layer" in k]
    non_ternary = {k: v.clone() for k, v in int8_model.items()
                   if not (v.dim() == 2 and "layer" in k) and "output.weight" not in k}
    workers = workers or max(1, (os.cpu_count() or 2) // 2)
    ternary = {}
    with ThreadPoolExecutor(max_workers=workers) as pool:
        for part in pool.map(convert_one_weight, tasks):
            ternary.update(part)
    return ternary, non_ternary


def convert_checkpoint(state: Dict[str, torch.Tensor], cfg: Optional[CheckpointShape] = None,
                       workers: Optional[int] = None):
    """bf16 state dict (keys as convert_back writes them, convert_TernaInfer.py:52-95) ->
    (bf16_model, ternary_result, non_ternary), the contents of the converter's three files."""
    bf16_model = convert_bitnet_checkpoint_to_bf16(state, cfg)
    ternary, non_ternary = compress_checkpoint(convert_bitnet_checkpoint_to_int8(state, cfg), workers)
    return bf16_model, ternary, non_ternary


def save_checkpoint(output_dir: str, bf16_model, ternary, non_ternary) -> None:
    os.makedirs(output_dir, exist_ok=True)
    torch.save(bf16_model, os.path.join(output_dir, CKPT_BF16))
    torch.save(ternary, os.path.join(output_dir, CKPT_TERNARY))
    torch.save(non_ternary, os.path.join(output_dir, CKPT_NON_TERNARY))


def load_checkpoint(ckpt_dir: str, bf16: bool = False) -> Dict[str, torch.Tensor]:
    """The dictionary the model constructors index (generate.py:64-71): the dense file, or the
    ternary and non-ternary files merged.  Tensors only (`weights_only=True`)."""
    load = lambda name: torch.load(os.path.join(ckpt_dir, name), map_location="cpu", weights_only=True)
    if bf16:
        return load(CKPT_BF16)
    return {**load(CKPT_TERNARY), **load(CKPT_NON_TERNARY)}


def main(argv=None) -> None:
    """Command line of the reference's converter (convert_TernaInfer.py:212-268): one .safetensors file in,
    the three .pt files out."""
    import argparse
    ap = argparse.ArgumentParser(description=main.__doc__)
    ap.add_argument("--safetensors_file", type=str, required=True)
    ap.add_argument("--output_dir", type=str, default="./checkpoints/")
    ap.add_argument("--workers", type=int, default=max(1, (os.cpu_count() or 2) // 2))
    args = ap.parse_args(argv)
    state = convert_back(args.safetensors_file)
    save_checkpoint(args.output_dir, *convert_checkpoint(state, workers=args.workers))
    print(f"Saved {CKPT_BF16}, {CKPT_TERNARY}, {CKPT_NON_TERNARY} to {args.output_dir}")


if __name__ == "__main__":
    main()
