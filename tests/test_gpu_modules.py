"""The call-site classes of the reference's model.py:96-153 and their bf16-activation siblings on the GPU:
SpBitLinear, BF16BitLinear (the reference's dense golden mode, `--BF16`), SpBitLinearBF16 and
TernaInfer_linear_bf16, each against the CPU oracle, and the sparse module against the dense one."""
import numpy as np
import pytest
import torch

from oracle import terna_oracle as O
from tests._util import check_against_fp64, make_bf16_activations, make_ternary

pytestmark = pytest.mark.gpu


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def checkpoint_entry(w, scales, key="l"):
    """What the converter writes for one linear: the four format tensors, the 4-slot bf16 weight_scale, and the
    dense bf16 matrix ternary * scale of the bf16 checkpoint (convert_TernaInfer.py:112-114, 159-194)."""
    import ternainfer_amd as T
    n = w.shape[0]
    vals, off, med, bm = T.compress_weight(torch.from_numpy(w))
    ws = T.pack_weight_scale([torch.tensor(v, dtype=torch.bfloat16) for v in scales])
    groups = O.ws_group_decode(np.arange(n), n, len(scales))
    dense = (torch.from_numpy(w).float() * ws.float()[torch.from_numpy(groups)][:, None]).to(torch.bfloat16)
    return {f"{key}.weight_compressed_val": vals, f"{key}.weight_TileOffsets_global": off,
            f"{key}.weight_TileOffsets_median": med, f"{key}.weight_bitmap": bm, f"{key}.weight_scale": ws,
            f"{key}.weight": dense}, ws


def _check(got_bits, ref, max_rel=1e-2, med_ulp_max=1):
    max_err, max_ref, med_ulp, _ = check_against_fp64(got_bits, ref)
    assert max_err <= max_rel * max_ref and med_ulp <= med_ulp_max, (max_err, max_ref, med_ulp)


@pytest.mark.parametrize("m,n,k,scales", [(5, 384, 256, [1.59375, 0.8125]), (8, 2560, 2560, [1.25]),
                                          (1, 3840, 2560, [0.75, 1.5, 1.125]), (96, 512, 320, [0.5])])
def test_bf16bitlinear_dense_mode_against_oracle_and_sparse_module(m, n, k, scales):
    """BF16BitLinear (model.py:135-153) within the bf16-GEMM bar of the float64 evaluation of its formula, and
    SpBitLinear on the compressed form of the same weights within a bf16 step or two of it: the dense mode is
    the reference's own golden for the sparse path (README `--BF16`)."""
    import ternainfer_amd as T
    w = make_ternary(n, k, 0.40, 700 + m + n)
    dic, ws = checkpoint_entry(w, scales)
    x_bits = make_bf16_activations(m, k, 710 + m + k)
    x = torch.from_numpy(x_bits.view(np.int16)).view(torch.bfloat16).cuda()
    print(f"[case] BF16BitLinear / SpBitLinear M={m} N={n} K={k} groups={len(scales)}", flush=True)
    dense_mod = T.BF16BitLinear(k, n, dic, "l")
    got = dense_mod(x)
    torch.cuda.synchronize()
    assert got.shape == (m, n) and got.dtype == torch.bfloat16
    ref = O.bf16_bitlinear_golden(x_bits, bits(dic["l.weight"]))
    _check(bits(got), ref)
    # the module's quantiser is the library's one definition
    q, s = dense_mod.quant_input(x)
    q_want, s_want = O.quant_input(x_bits)
    assert (q.cpu().numpy() == q_want).all() and (bits(s).reshape(-1) == s_want).all()
    sparse = T.SpBitLinear(k, n, dic, "l")(x)
    torch.cuda.synchronize()
    _check(bits(sparse), ref)
    # bit-exact against the integer oracle with the epilogue rule the row count selects
    want = O.spmm_i8(q_want, w, s_want, bits(ws), len(scales), 0 if max(8, 1 << (m - 1).bit_length()) <= 64 else 1)
    assert (bits(sparse) == want).all()


@pytest.mark.parametrize("shape,n,k,scales", [((3, 320), 256, 320, [0.7, 1.9]), ((2, 5, 320), 256, 320, [1.3]),
                                              ((8, 2560), 2560, 2560, [1.37]), ((300, 192), 384, 192, [0.9, 1.1])])
def test_spbitlinear_bf16_module_and_call_site(shape, n, k, scales):
    """SpBitLinearBF16 and TernaInfer_linear_bf16 (auto / forced routes; 2-D and 3-D inputs keep their leading
    dimensions) against the float64 golden of the bf16-activation family."""
    import ternainfer_amd as T
    w = make_ternary(n, k, 0.40, 720 + n + len(shape))
    dic, ws = checkpoint_entry(w, scales)
    m = int(np.prod(shape[:-1]))
    x_bits = make_bf16_activations(m, k, 730 + m, outlier_frac=0.01 if m > 64 else 0.0)
    x = torch.from_numpy(x_bits.view(np.int16)).view(torch.bfloat16).reshape(shape).cuda()
    scale = ws.float().numpy()
    ref = O.spmm_bf16_golden(x_bits, w, scale[:len(scales)], len(scales))
    print(f"[case] SpBitLinearBF16 / TernaInfer_linear_bf16 shape={shape} N={n} K={k}", flush=True)
    mod = T.SpBitLinearBF16(k, n, dic, "l")
    assert mod.ws_num == len(scales)
    got = mod(x)
    torch.cuda.synchronize()
    assert tuple(got.shape) == tuple(shape[:-1]) + (n,) and got.dtype == torch.bfloat16
    _check(bits(got).reshape(m, n), ref)
    dev = lambda t: t.cuda()
    for route in ("auto", "decode", "prefill"):
        out = T.TernaInfer_linear_bf16(x, dev(dic["l.weight_compressed_val"]), dev(dic["l.weight_TileOffsets_global"]),
                                       dev(dic["l.weight_TileOffsets_median"]), dev(dic["l.weight_bitmap"]),
                                       dev(ws.float()), len(scales), n, route=route)
        torch.cuda.synchronize()
        assert tuple(out.shape) == tuple(shape[:-1]) + (n,)
        _check(bits(out).reshape(m, n), ref)
