"""Run under pytest by tests/test_gpu_parity.py::test_tile_and_path_overrides in a child process whose
environment pins one of the library's tuning overrides (they are read once per process): large-M
parity of both families on shapes with ragged M, N tails and odd / even tile counts, the small-M
kernels on both layouts, and the decode-step kernels (prologue inside the linear, attention)."""
import sys

import numpy as np
import torch

from oracle import terna_oracle as O
from tests._util import DeviceFormat, make_bf16_activations, make_int8_activations, make_ternary
from tests.test_gpu_parity import WS, _check_bf16, repack, run_bf16_packed, run_i8_packed
from ternainfer_amd import _lib


def main() -> int:
    lib = _lib.load()
    co = O.COracle()
    for m, n, k in [(100, 320, 192), (300, 512, 320), (65, 256, 64), (256, 3840, 128), (512, 384, 128), (1024, 320, 64)]:
        w = make_ternary(n, k, 0.40, 900 + m + n)
        packed = repack(lib, DeviceFormat(w))
        xq, s = make_int8_activations(m, k, 901 + m)
        print(f"[case] override check m={m} n={n} k={k}", flush=True)
        if not (run_i8_packed(lib, packed, n, xq, s, WS, 1, 1) == O.spmm_i8(xq, w, s, WS, 1, 1)).all():
            print("int8 mismatch", m, n, k)
            return 1
        x = make_bf16_activations(m, k, 902 + m, outlier_frac=0.01)
        scale = np.array([0.7], np.float32)
        _check_bf16(run_bf16_packed(lib, packed, n, x, scale, 1, 1), co.spmm_bf16(x, w, scale, 1))
    # split-K of the MFMA-tiled kernel with scratch memory (TERNASPMM_PREFILL_SPLITS forces the split count)
    from tests.test_gpu_parity import _run_packed_ws
    for m, n, k in [(100, 256, 2048), (300, 384, 832)]:
        w = make_ternary(n, k, 0.40, 905 + m + n)
        packed = repack(lib, DeviceFormat(w))
        work = torch.empty(8 * m * n * 4, dtype=torch.int8, device="cuda")
        xq, s = make_int8_activations(m, k, 906 + m)
        if not (_run_packed_ws(lib, "int8", packed, n, xq, s, WS, 2, 8, work) == O.spmm_i8(xq, w, s, WS, 2, 1)).all():
            print("int8 split-K mismatch", m, n, k)
            return 1
        x = make_bf16_activations(m, k, 907 + m, outlier_frac=0.01)
        scale = np.array([0.7, 1.1], np.float32)
        _check_bf16(_run_packed_ws(lib, "bf16", packed, n, x, None, scale, 2, 1, work), co.spmm_bf16(x, w, scale, 2))
    from tests.test_gpu_parity import run_bf16, run_i8
    for m, n, k in [(8, 320, 192), (16, 256, 64), (1, 8256, 128)]:      # small-M kernels, both layouts
        w = make_ternary(n, k, 0.40, 910 + m + n)
        fmt = DeviceFormat(w)
        packed = repack(lib, fmt)
        xq, s = make_int8_activations(m, k, 911 + m)
        x = make_bf16_activations(m, k, 912 + m)
        scale = np.array([0.7], np.float32)
        want = O.spmm_i8(xq, w, s, WS, 1, 0)
        if not ((run_i8_packed(lib, packed, n, xq, s, WS, 1) == want).all() and (run_i8(lib, fmt, xq, s, WS, 1) == want).all()):
            print("int8 small-M mismatch", m, n, k)
            return 1
        gold = co.spmm_bf16(x, w, scale, 1)
        _check_bf16(run_bf16_packed(lib, packed, n, x, scale, 1), gold)
        _check_bf16(run_bf16(lib, fmt, x, scale, 1), gold)
    # the decode-step kernels behind their overrides: prologue inside the linear, single-token attention
    from tests import test_gpu_prologue as P
    for m, n, k, ws_num, res in [(1, 13824, 2560, 2, True), (8, 13824, 2560, 2, True), (1, 2560, 2560, 1, False)]:
        P.test_fused_prologue_linear(lib, m, n, k, ws_num, res)
    P.test_decode_attention(lib, 1, 20, 5, 128, 1024, 1000, True)
    P.test_decode_attention(lib, 2, 4, 2, 64, 300, 290, True)
    P.test_rope_decode_attention_equals_the_two_launches(lib, 1, 20, 5, 128, 2048, 1500, 1, True)
    torch.cuda.synchronize()
    print("override check ok")
    return 0


if __name__ == "__main__":
    sys.exit(main())
