"""The C-ABI library loads without a GPU and exports every symbol include/ternaspmm.h declares."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ternaspmm.h")

REFERENCE_SYMBOLS = ["checkLastCudaError", "bitlinear_TernaSpMM", "bitlinear_TernaSpMM_decode",
                     "bitlinear_TernaSpMM_prefill", "bitlinear_TernaSpMM_benchmark", "reorder_WT_h",
                     "convert_reorderd", "gpu_sleep"]


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"^\s*(?:const\s+)?[A-Za-z_][\w\s\*]*?\b([A-Za-z_]\w*)\s*\(", text, flags=re.M)


def test_header_declares_the_reference_symbols():
    names = declared_symbols()
    for sym in REFERENCE_SYMBOLS:
        assert sym in names, sym


def test_library_exports_every_declared_symbol():
    from ternainfer_amd import _lib
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 15
    for sym in names:
        assert hasattr(lib, sym), f"{sym} declared in include/ternaspmm.h but not exported"
        assert sym in _lib.PROTOTYPES, f"{sym} has no ctypes prototype"
    assert set(_lib.PROTOTYPES) == set(names)


def test_version_string():
    from ternainfer_amd import _lib
    assert _lib.load().ternaspmm_version().startswith(b"ternaspmm-gfx950")


def test_missing_library_fails_loudly(monkeypatch):
    from ternainfer_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libternaspmm.so")
    with pytest.raises(ImportError):
        _lib.load()


def test_encode_sizes_rejects_bad_shapes():
    from ternainfer_amd import _lib
    lib = _lib.load()
    out = (ctypes.c_int64 * 4)()
    ptrs = [ctypes.byref(out, 8 * j) for j in range(4)]
    assert lib.ternaspmm_encode_sizes(64, 100, *ptrs) == -1
    assert lib.ternaspmm_encode_sizes(128, 192, *ptrs) == 0
    assert list(out) == [128 * 192 // 64, 128 * 192 // 4096 + 1, 3 * 128 * 192 // 4096, 128 * 192 // 32]


def test_unsupported_shapes_are_refused_before_any_device_work():
    """A shape the format cannot express, and a K too deep for int8 activations on the P2 layout (its 32-bit
    accumulator holds 64 times the sum), print a message and return without a launch (the reference's
    unsupported-batch branch, TernaSpMM_API.cuh:117-120): no pointer is touched, so this runs without a GPU."""
    import subprocess
    import sys
    code = ("from ternainfer_amd import _lib\n"
            "lib = _lib.load()\n"
            "lib.bitlinear_TernaSpMM_packed(None, None, None, None, None, 1, 1, 64, 100, 0, None)\n"
            "lib.bitlinear_TernaSpMM_packed(None, None, None, None, None, 1, 1, 64, 262144, 0, None)\n"
            "lib.bitlinear_TernaSpMM(None, None, None, None, None, None, None, None, 1, 8, 64, 262144, 1, None, None)\n"
            "lib.bitlinear_TernaSpMM_bf16_packed(None, None, None, None, 5, 1, 64, 64, 0, None)\n"
            "print('returned', flush=True)\n")
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "unsupported shape M=1 N=64 K=100" in r.stdout
    assert r.stdout.count("unsupported K=262144 with int8 activations (need K <= 262080)") == 2
    assert "unsupported ws_num=5" in r.stdout
    assert r.stdout.rstrip().endswith("returned")


def test_host_side_size_and_policy_functions():
    """Functions that only compute on the host: buffer sizes and the recommended split count of the attention."""
    from ternainfer_amd import _lib
    lib = _lib.load()
    assert lib.ternaspmm_packed_bytes(2560, 6912) == 2560 * 6912 // 4
    assert lib.ternaspmm_packed_bytes(2560, 100) < 0
    assert lib.ternaspmm_attention_partial_bytes(1, 20, 128) == 4 * (20 * 16 + 20 * 8 * 128)
    assert lib.ternaspmm_attention_partial_bytes(0, 20, 128) == -1
    assert lib.ternaspmm_attention_partial_splits(1, 20, 384) == 4       # up to 1024 slots: four splits
    assert lib.ternaspmm_attention_partial_splits(1, 20, 4096) == 8      # beyond: eight
    assert lib.ternaspmm_attention_partial_splits(8, 20, 384) == 1       # the heads fill the chip anyway
    assert lib.ternaspmm_attention_partial_splits(8, 20, 2048) == 4      # ... but a long cache is split all the same
    assert lib.ternaspmm_attention_partial_splits(64, 20, 2048) == 1     # up to about eight workgroups per CU
    assert lib.ternaspmm_attention_partial_splits(1, 20, 32) == 1        # a split must keep two tiles
    assert lib.ternaspmm_attention_partial_splits(1, 20, 64) == 2
    assert lib.ternaspmm_attention_partial_splits(1, 20, 128) == 4
    assert lib.ternaspmm_attention_workspace_bytes(1, 20, 128) > 0
    # knowing the kv heads: several sequences with 2 or 4 heads per kv head split from 512 slots on (one workgroup per kv head)
    assert lib.ternaspmm_attention_partial_splits_kv(8, 20, 5, 384) == 1
    assert lib.ternaspmm_attention_partial_splits_kv(8, 20, 5, 728) == 4
    assert lib.ternaspmm_attention_partial_splits_kv(16, 20, 5, 728) == 2
    assert lib.ternaspmm_attention_partial_splits_kv(8, 20, 5, 2048) == lib.ternaspmm_attention_partial_splits(8, 20, 2048)
    assert lib.ternaspmm_attention_partial_splits_kv(1, 20, 5, 728) == lib.ternaspmm_attention_partial_splits(1, 20, 728)
    assert lib.ternaspmm_attention_partial_splits_kv(8, 20, 20, 728) == lib.ternaspmm_attention_partial_splits(8, 20, 728)
    assert lib.ternaspmm_attention_partial_splits_kv(8, 20, 3, 728) == -1
    # refused on the host, nothing enqueued: split counts and row lengths the merge + norm + quantise launch does not take
    assert lib.ternaspmm_attention_merge_rmsnorm_quant(None, 3, None, 1e-5, None, None, None, 8, 20, 128, None) == -1
    assert lib.ternaspmm_attention_merge_rmsnorm_quant(None, 4, None, 1e-5, None, None, None, 8, 40, 128, None) == -1


def test_python_wrappers_refuse_mismatched_tensors_on_the_host():
    """The library takes pointers and sizes on trust; the Python wrappers check element counts first, so that a
    tensor with too few rows raises here instead of being read or written past its end on the GPU.  (CPU tensors:
    the checks run before anything touches a device.)"""
    import torch
    from ternainfer_amd import linear as L
    x = torch.zeros(8, 2560, dtype=torch.bfloat16)
    one_row = torch.zeros(1, 2560, dtype=torch.bfloat16)
    w = torch.zeros(2560, dtype=torch.bfloat16)
    ws = torch.zeros(4, dtype=torch.bfloat16)
    packed = torch.zeros(2560 * 2560 // 4, dtype=torch.int8)
    with pytest.raises(ValueError, match="residual"):
        L.rmsnorm_quant(x, w, 1e-5, residual=one_row)
    with pytest.raises(ValueError, match="residual"):
        L.rmsnorm_linear_packed(x, w, 1e-5, packed, ws, 1, 2560, residual=one_row)
    with pytest.raises(ValueError, match="norm_weight"):
        L.rmsnorm_linear_packed(x, w[:100], 1e-5, packed, ws, 1, 2560)
    with pytest.raises(ValueError, match="too small"):
        L.rmsnorm_linear_packed(x, w, 1e-5, packed[:1000], ws, 1, 2560)
    with pytest.raises(ValueError, match="s has"):
        L.TernaInfer_linear_packed(torch.zeros(8, 2560, dtype=torch.int8), packed, torch.zeros(1, dtype=torch.bfloat16), ws, 1, 2560)
    with pytest.raises(ValueError, match="weight"):
        L.relu2_mul_rmsnorm_quant(torch.zeros(2, 2 * 6912, dtype=torch.bfloat16), w, 1e-5)
    with pytest.raises(ValueError, match="does not hold"):
        L.attention_merge_rmsnorm_linear_packed(torch.zeros(1000, dtype=torch.float32), 4, 20, 128, w, 1e-5, packed, ws, 1, 2560,
                                                sequences=8)
