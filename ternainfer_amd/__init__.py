"""MI355X-native TernaSpMM: ternary-weight sparse x dense matmul behind libternaspmm.so."""
from . import _lib  # noqa: F401
from .convert_utils import (  # noqa: F401
    CheckpointShape, compress_checkpoint, compress_weight, convert_back, convert_bitnet_checkpoint_to_bf16,
    convert_bitnet_checkpoint_to_int8, convert_checkpoint, load_checkpoint, pack_weight_scale, quant_weight_int8,
    reorder_weight, save_checkpoint)
from .linear import (  # noqa: F401
    BF16BitLinear, SpBitLinear, argmax_rows, greedy_step, greedy_step_state, lm_head, SpBitLinearBF16, TernaInfer_linear, TernaInfer_linear_bf16,
    TernaInfer_linear_packed, fused_linear, get_global_workspace, interleave_gate_up, row_stats, relu2_mul_rmsnorm_linear_packed, relu2_mul_rmsnorm_quant, repack_weight, rmsnorm_linear_packed, rmsnorm_quant)

__version__ = "0.1"
