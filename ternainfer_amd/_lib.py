"""ctypes loader for ``kernels/libternaspmm.so`` (the C-ABI boundary of the TernaSpMM path).

The reference binds the library with ``ctypes.CDLL('./kernels/libternaspmm.so')`` and no
prototypes (model.py:21).  Here the path is resolved from the package location so that the
import works from any directory, and prototypes are declared so that a wrong argument count
fails in Python instead of corrupting the call.  There is no fallback: if the library has
not been built the import raises.
"""
from __future__ import annotations

import ctypes
import os

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.environ.get("TERNASPMM_LIB", os.path.join(_ROOT, "kernels", "libternaspmm.so"))

_vp, _ci = ctypes.c_void_p, ctypes.c_int
_i8_args = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp, _vp]
_bf16_args = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp, _vp]

#: every symbol include/ternaspmm.h declares -> (argtypes, restype)
PROTOTYPES = {
    "checkLastCudaError": ([_ci], None),
    "bitlinear_TernaSpMM": (_i8_args, None),
    "bitlinear_TernaSpMM_decode": (_i8_args, None),
    "bitlinear_TernaSpMM_prefill": (_i8_args, None),
    "bitlinear_TernaSpMM_benchmark": ([_ci, _ci, _ci] + _i8_args, None),
    "reorder_WT_h": ([_vp, _vp, _ci, _ci], None),
    "convert_reorderd": ([_vp, _ci, _ci, _ci, _ci, _ci, _ci, _ci, _ci, _vp, _vp, _vp, _vp, _vp], _ci),
    "gpu_sleep": ([ctypes.c_double, _vp], None),
    "bitlinear_TernaSpMM_bf16": (_bf16_args, None),
    "bitlinear_TernaSpMM_bf16_decode": (_bf16_args, None),
    "bitlinear_TernaSpMM_bf16_prefill": (_bf16_args, None),
    "ternaspmm_encode_sizes": ([_ci, _ci, _vp, _vp, _vp, _vp], _ci),
    "ternaspmm_encode_i8": ([_vp, _ci, _ci, _vp, _vp, _vp, _vp], ctypes.c_int64),
    "ternaspmm_decompress_bf16": ([_vp, _vp, _vp, _vp, _vp, _ci, _ci, _vp], None),
    "ternaspmm_packed_bytes": ([_ci, _ci], ctypes.c_int64),
    "ternaspmm_repack": ([_vp, _vp, _vp, _vp, _vp, _ci, _ci, _vp], None),
    "bitlinear_TernaSpMM_bf16_packed": ([_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp], None),
    "bitlinear_TernaSpMM_packed": ([_vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp], None),
    "bitlinear_TernaSpMM_bf16_packed_ws": ([_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp, ctypes.c_longlong, _vp], None),
    "bitlinear_TernaSpMM_packed_ws": ([_vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp, ctypes.c_longlong, _vp], None),
    "ternaspmm_rmsnorm_quant": ([_vp, _vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _ci, _ci, _vp], None),
    "ternaspmm_relu2_mul_rmsnorm_quant": ([_vp, _vp, ctypes.c_float, _vp, _vp, _vp, _ci, _ci, _vp], None),
    "bitlinear_TernaSpMM_packed_fused": ([_vp, _vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _ci, _vp, _vp, _ci, _ci, _ci, _vp],
                                         ctypes.c_int),
    "bitlinear_TernaSpMM_packed_fused_attn": ([_vp, _ci, _ci, _vp, ctypes.c_float, _vp, _vp, _vp, _ci, _vp, _vp, _ci, _ci, _ci, _vp],
                                              ctypes.c_int),
    "bitlinear_TernaSpMM_packed_fused_glu": ([_vp, _vp, ctypes.c_float, _vp, _vp, _vp, _ci, _vp, _vp, _ci, _ci, _ci, _vp],
                                             ctypes.c_int),
    "ternaspmm_rope_decode_attention_prefetch": ([_vp] * 4 + [_ci] + [_vp] * 3 + [_ci] * 5 + [ctypes.c_float, _ci, _vp, _vp, _vp, _vp, _ci, _vp], None),
    "ternaspmm_greedy_step_state_bytes": ([_ci], ctypes.c_size_t),
    "ternaspmm_greedy_step_bf16": ([_vp, _vp, _vp, _ci, _vp, _vp, _ci, _ci, _vp], None),
    "ternaspmm_lm_head_bf16": ([_vp, _vp, _vp, _ci, _ci, _ci, _vp], None),
    "ternaspmm_argmax_bf16": ([_vp, _vp, _ci, _ci, _vp], None),
    "ternaspmm_attention_partial_bytes": ([_ci] * 3, ctypes.c_longlong),
    "ternaspmm_attention_partial_splits": ([_ci] * 3, ctypes.c_int),
    "ternaspmm_attention_partial_splits_kv": ([_ci] * 4, ctypes.c_int),
    "ternaspmm_rope_decode_attention_partial": ([_vp] * 4 + [_ci] + [_vp] * 3 + [_ci] * 6 + [ctypes.c_float, _ci, _vp, _vp, _vp, _ci, _vp], None),
    "ternaspmm_attention_merge": ([_vp, _ci, _vp, _ci, _ci, _ci, _vp], None),
    "ternaspmm_attention_merge_rmsnorm_quant": ([_vp, _ci, _vp, ctypes.c_float, _vp, _vp, _vp, _ci, _ci, _ci, _vp], ctypes.c_int),
    "ternaspmm_rope_kv_store": ([_vp] * 4 + [_ci] + [_vp] * 3 + [_ci] * 7 + [_vp], None),
    "ternaspmm_rope_decode_attention_stats": ([_vp] * 4 + [_ci] + [_vp] * 3 + [_ci] * 5 + [ctypes.c_float, _ci, _vp, _vp, _vp], ctypes.c_int),
    "ternaspmm_rope_decode_attention": ([_vp] * 4 + [_ci] + [_vp] * 3 + [_ci] * 5 + [ctypes.c_float, _ci, _vp, _vp], None),
    "ternaspmm_decode_attention": ([_vp] * 4 + [_ci, _vp] + [_ci] * 5 + [ctypes.c_float, _vp, _vp], None),
    "ternaspmm_prefill_attention": ([_vp] * 4 + [_ci, _vp] + [_ci] * 6 + [ctypes.c_float, _vp], None),
    "ternaspmm_decode_attention_static": ([_vp] * 4 + [_ci, _vp] + [_ci] * 5 + [ctypes.c_float, _vp], ctypes.c_int),
    "ternaspmm_attention_workspace_bytes": ([_ci, _ci, _ci], ctypes.c_longlong),
    "ternaspmm_probe_empty": ([_vp], None),
    "ternaspmm_probe_empty_shape": ([_ci, _ci, _ci, _vp], _ci),
    "ternaspmm_probe_read": ([_vp, ctypes.c_longlong, _vp, _vp], None),
    "ternaspmm_probe_read_grid": ([_vp, ctypes.c_longlong, _vp, _ci, _vp], _ci),
    "ternaspmm_probe_copy": ([_vp, _vp, ctypes.c_longlong, _vp], None),
    "ternaspmm_probe_barrier_state_bytes": ([], ctypes.c_size_t),
    "ternaspmm_probe_barrier": ([_vp, _ci, _ci, ctypes.c_uint, _vp], ctypes.c_int),
    "ternaspmm_repack_cache_clear": ([], None),
    "ternaspmm_repack_cache_enable": ([_ci], _ci),
    "ternaspmm_repack_cache_limit": ([ctypes.c_longlong], ctypes.c_longlong),
    "ternaspmm_repack_cache_stats": ([_vp], None),
    "ternaspmm_plan_reference_call": ([_ci] * 6 + [_vp, _ci, _vp], _ci),
    "ternaspmm_quant_mode": ([_ci], _ci),
    "ternaspmm_fused_linear": ([_vp, _vp], _ci),
    "ternaspmm_quant_from_stats": ([_vp, _vp, _ci, _vp, ctypes.c_float, _vp, _vp, _ci, _ci, _vp], _ci),
    "ternaspmm_row_stats_count": ([_ci], _ci),
    "ternaspmm_row_stats": ([_vp, _vp, _vp, _ci, _ci, _vp], _ci),
    "ternaspmm_interleave_gate_up": ([_vp, _vp, _ci, _ci, _vp], _ci),
    "ternaspmm_step_inputs": ([_vp, _vp, _ci, _vp, _ci, _ci, _vp, _ci, _ci, _vp, _vp, _vp, _vp, _ci, _vp], _ci),
    "ternaspmm_version": ([], ctypes.c_char_p),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library once and attach prototypes.  Raises if it is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: build it with `bash kernels/compile.sh` "
                "(hipcc --offload-arch=gfx950); there is no fallback path")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (argtypes, restype) in PROTOTYPES.items():
            fn = getattr(lib, name)          # AttributeError if the symbol is not exported
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = lib
    return _lib
