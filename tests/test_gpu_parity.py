"""Parity of the HIP path against the CPU oracle, through the C ABI, on a real MI355X.

  int8 family : bit-exact (integer accumulate + the reference's fp32 epilogue arithmetic)
  bf16 family : max|err| <= 1e-2 * max|ref| and median error <= 1 bf16 ULP against the fp64 golden
  format      : device decompression of the compressed format is bit-exact
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from oracle import terna_oracle as O
from tests._util import (DeviceFormat, check_against_fp64, make_bf16_activations, make_int8_activations,
                         make_row_skewed, make_ternary, seed_for, vp)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    from ternainfer_amd import _lib
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return _lib.load()


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


_CANARY = 1 << 20


class _Workspace:
    """Exactly the bytes the reference itself would write for this call -- SPLIT_K int32 planes of M x N on its decode
    path (tests/test_kernel.cu:331), a dense int8 N x K matrix on its prefill path (model.py:34-42) -- followed by a
    canary region that must come back untouched."""

    def __init__(self, entry, m, n, k, split_k):
        prefill_path = entry.endswith("_prefill") or (not entry.endswith("_decode") and m > 64)
        self.bytes = n * k if prefill_path else 4 * m * n * split_k
        self.buf = torch.full((self.bytes + _CANARY,), 0x5A, dtype=torch.int8, device="cuda")

    def check(self):
        assert bool((self.buf[self.bytes:] == 0x5A).all()), "the call wrote past the workspace the reference guarantees"


def _workspace(m, n, k):
    """Room for both of the reference's uses of its workspace (model.py:34-42): callers that do not go through run_i8 /
    run_bf16."""
    return torch.empty(max(4 * m * n * 7, n * k) + 256, dtype=torch.int8, device="cuda")


def run_i8(lib, fmt, xq, s_bits, ws_bits, ws_num, entry="bitlinear_TernaSpMM", workspace=True):
    m, k = xq.shape
    x = torch.from_numpy(xq).cuda()
    s = torch.from_numpy(s_bits.view(np.int16)).cuda()
    ws = torch.from_numpy(ws_bits.view(np.int16)).cuda()
    out = torch.full((m, fmt.n), -1, dtype=torch.int16, device="cuda")      # poison: must be overwritten
    work = _Workspace(entry, m, fmt.n, k, 7) if workspace else None
    print(f"[case] {entry} M={m} N={fmt.n} K={k} ws_num={ws_num} workspace={workspace}", flush=True)
    getattr(lib, entry)(vp(x), vp(fmt.bm), vp(fmt.off), vp(fmt.med), vp(fmt.vals), vp(out), vp(s), vp(ws),
                        ws_num, m, fmt.n, k, 7, vp(work.buf) if workspace else None, _stream())
    torch.cuda.synchronize()
    if workspace:
        work.check()
    return out.cpu().numpy().view(np.uint16)


def run_bf16(lib, fmt, x_bits, scale, ws_num, entry="bitlinear_TernaSpMM_bf16", workspace=False, split_k=1):
    m, k = x_bits.shape
    x = torch.from_numpy(x_bits.view(np.int16)).cuda()
    sc = torch.from_numpy(scale).cuda()
    out = torch.full((m, fmt.n), -1, dtype=torch.int16, device="cuda")
    work = _Workspace(entry, m, fmt.n, k, split_k) if workspace else None
    print(f"[case] {entry} M={m} N={fmt.n} K={k} ws_num={ws_num} workspace={workspace}", flush=True)
    getattr(lib, entry)(vp(x), vp(fmt.bm), vp(fmt.off), vp(fmt.med), vp(fmt.vals), vp(out), vp(sc), ws_num,
                        m, fmt.n, k, split_k, vp(work.buf) if workspace else None, _stream())
    torch.cuda.synchronize()
    if workspace:
        work.check()
    return out.cpu().numpy().view(np.uint16)


def repack(lib, fmt):
    """Reference format -> P2 on the device."""
    nbytes = lib.ternaspmm_packed_bytes(fmt.n, fmt.k)
    assert nbytes == fmt.n * fmt.k // 4
    packed = torch.full((nbytes // 4,), -1, dtype=torch.int32, device="cuda")
    print(f"[case] ternaspmm_repack N={fmt.n} K={fmt.k}", flush=True)
    lib.ternaspmm_repack(vp(fmt.bm), vp(fmt.off), vp(fmt.med), vp(fmt.vals), vp(packed), fmt.n, fmt.k, _stream())
    torch.cuda.synchronize()
    return packed


def run_bf16_packed(lib, packed, n, x_bits, scale, ws_num, route=0):
    m, k = x_bits.shape
    x = torch.from_numpy(x_bits.view(np.int16)).cuda()
    sc = torch.from_numpy(scale).cuda()
    out = torch.full((m, n), -1, dtype=torch.int16, device="cuda")
    print(f"[case] bitlinear_TernaSpMM_bf16_packed M={m} N={n} K={k} ws_num={ws_num} route={route}", flush=True)
    lib.bitlinear_TernaSpMM_bf16_packed(vp(x), vp(packed), vp(out), vp(sc), ws_num, m, n, k, route, _stream())
    torch.cuda.synchronize()
    return out.cpu().numpy().view(np.uint16)


def run_i8_packed(lib, packed, n, xq, s_bits, ws_bits, ws_num, route=0):
    m, k = xq.shape
    x = torch.from_numpy(xq).cuda()
    s = torch.from_numpy(s_bits.view(np.int16)).cuda()
    ws = torch.from_numpy(ws_bits.view(np.int16)).cuda()
    out = torch.full((m, n), -1, dtype=torch.int16, device="cuda")
    print(f"[case] bitlinear_TernaSpMM_packed M={m} N={n} K={k} ws_num={ws_num} route={route}", flush=True)
    lib.bitlinear_TernaSpMM_packed(vp(x), vp(packed), vp(out), vp(s), vp(ws), ws_num, m, n, k, route, _stream())
    torch.cuda.synchronize()
    return out.cpu().numpy().view(np.uint16)


WS = O.f32_to_bf16_bits(np.array([0.8125, 1.59375, 2.71875, 0.3359375], np.float32))


# ------------------------------------------------------------------------------- format
@pytest.mark.parametrize("kind", ["iid40", "iid45", "skewed", "dense", "empty", "sparse97"])
def test_device_decompress_is_bit_exact(lib, kind):
    n, k = 256, 320
    w = {"iid40": lambda: make_ternary(n, k, 0.40, 1), "iid45": lambda: make_ternary(n, k, 0.45, 2),
         "skewed": lambda: make_row_skewed(n, k, 3), "dense": lambda: make_ternary(n, k, 0.0, 4),
         "empty": lambda: np.zeros((n, k), np.int8), "sparse97": lambda: make_ternary(n, k, 0.97, 5)}[kind]()
    fmt = DeviceFormat(w)
    dense = torch.full((n, k), 0x7FC0, dtype=torch.int16, device="cuda")
    print(f"[case] decompress {kind} N={n} K={k}", flush=True)
    lib.ternaspmm_decompress_bf16(vp(fmt.bm), vp(fmt.off), vp(fmt.med), vp(fmt.vals), vp(dense), n, k, _stream())
    torch.cuda.synchronize()
    got = O.bf16_bits_to_f32(dense.cpu().numpy().view(np.uint16))
    assert (got == w.astype(np.float32)).all()


def test_device_decompress_full_size_round_trip(lib):
    """BitNet-2B gate+up shape: decompress(encode(W)) == W on the device."""
    n, k = 13824, 2560
    w = make_ternary(n, k, 0.40, seed_for(2, 3))
    fmt = DeviceFormat(w)
    dense = torch.empty((n, k), dtype=torch.bfloat16, device="cuda")
    lib.ternaspmm_decompress_bf16(vp(fmt.bm), vp(fmt.off), vp(fmt.med), vp(fmt.vals), vp(dense), n, k, _stream())
    torch.cuda.synchronize()
    assert torch.equal(dense.cpu(), torch.from_numpy(w).to(torch.bfloat16))


# ------------------------------------------------------------------------------- int8 family
@pytest.mark.parametrize("m", [1, 8, 16, 24, 32, 64])
@pytest.mark.parametrize("n,k,ws_num", [(128, 192, 1), (256, 320, 2), (256, 64, 4)])
def test_int8_small_m_bit_exact(lib, coracle, m, n, k, ws_num):
    w = make_ternary(n, k, 0.40, 10 + m + n)
    fmt = DeviceFormat(w)
    xq, s = make_int8_activations(m, k, 20 + m + k)
    got = run_i8(lib, fmt, xq, s, WS, ws_num)
    want = coracle.spmm_i8(xq, w, s, WS, ws_num, 0)
    assert (got == want).all()


@pytest.mark.parametrize("entry,mode,m", [("bitlinear_TernaSpMM_decode", 0, 8), ("bitlinear_TernaSpMM_decode", 0, 128),
                                          ("bitlinear_TernaSpMM_prefill", 1, 8), ("bitlinear_TernaSpMM_prefill", 1, 128),
                                          ("bitlinear_TernaSpMM", 1, 128), ("bitlinear_TernaSpMM", 1, 200)])
def test_int8_forced_paths_follow_their_epilogue(lib, coracle, entry, mode, m):
    n, k = 384, 256
    w = make_ternary(n, k, 0.40, 31)
    fmt = DeviceFormat(w)
    xq, s = make_int8_activations(m, k, 32 + m)
    s = s.copy()
    if mode == 1:
        s[m // 2] = 0                     # prefill rule: coefficient 0 where s == 0
    got = run_i8(lib, fmt, xq, s, WS, 3, entry)
    want = coracle.spmm_i8(xq, w, s, WS, 3, mode)
    if mode == 0:
        assert (got == want).all()
    else:
        row = m // 2
        keep = np.arange(m) != row
        assert (got[keep] == want[keep]).all()
        assert not (got[row] & 0x7FFF).any() and (got[row] == want[row]).all()


def test_int8_qkv_groups_bit_exact(lib, coracle):
    """N = 3840 with three scales: the 2560 / 640 / 640 split of the fused QKV matrix."""
    n, k, m = 3840, 256, 8
    w = make_ternary(n, k, 0.40, 41)
    fmt = DeviceFormat(w)
    xq, s = make_int8_activations(m, k, 42)
    got = run_i8(lib, fmt, xq, s, WS, 3)
    assert (got == coracle.spmm_i8(xq, w, s, WS, 3, 0)).all()


def test_int8_reference_test_construction(lib):
    """tests/test_kernel.cu 8 2560 2560 45 7: x == 1, unit scales, ws_num = 4 -> exact row sums of W."""
    n = k = 2560
    m = 8
    w = make_ternary(n, k, 0.45, seed_for(1, 0))
    fmt = DeviceFormat(w)
    x = np.ones((m, k), np.int8)
    one = O.f32_to_bf16_bits(np.ones(4, np.float32))
    got = run_i8(lib, fmt, x, one[:1].repeat(m), one, 4)
    want = O.f32_to_bf16_bits(np.tile(w.sum(axis=1, dtype=np.int64).astype(np.float32), (m, 1)))
    assert (got == want).all()


@pytest.mark.parametrize("n,k", [(3840, 2560), (2560, 2560), (13824, 2560), (2560, 6912)])
@pytest.mark.parametrize("m", [1, 8, 16])
def test_int8_2b_layer_shapes_bit_exact(lib, m, n, k):
    w = make_ternary(n, k, 0.40, seed_for(2, n % 7))
    fmt = DeviceFormat(w)
    xq, s = make_int8_activations(m, k, seed_for(2, 10 + m))
    ws_num = 3 if n == 3840 else (2 if n == 13824 else 1)
    mp = max(8, 1 << (m - 1).bit_length())          # the call site pads rows (model.py:64)
    xq_p = np.concatenate([xq, np.zeros((mp - m, k), np.int8)])
    s_p = np.concatenate([s, O.f32_to_bf16_bits(np.ones(mp - m, np.float32))])
    got = run_i8(lib, fmt, xq_p, s_p, WS, ws_num)[:m]
    want = O.spmm_i8(xq, w, s, WS, ws_num, 0)
    assert (got == want).all()


# ------------------------------------------------------------------------------- bf16 family
def _assert_negation_symmetric(out_bits, out_of_negated_x_bits):
    """out(-x) == -out(x): exactly on all but a sliver of the outputs, and there to within one bf16
    step of the value (or of the cancellation noise floor for sums that nearly cancel) -- the
    matrix cores' internal fp32 summation is not exactly sign-symmetric."""
    a = O.bf16_bits_to_f32(out_bits).astype(np.float64)
    b = O.bf16_bits_to_f32(out_of_negated_x_bits).astype(np.float64)
    diff = np.abs(a + b)
    assert (diff != 0).mean() < 1e-4, float((diff != 0).mean())
    assert (diff <= 2.0 ** -7 * np.abs(a) + 1e-4 * np.abs(a).max()).all(), float(diff.max())


def _check_bf16(got, ref):
    max_err, max_ref, med_ulp, max_ulp = check_against_fp64(got, ref)
    assert max_err <= 1e-2 * max_ref, (max_err, max_ref)
    assert med_ulp <= 1, med_ulp
    return max_err / max_ref, med_ulp, max_ulp


@pytest.mark.parametrize("m", [1, 3, 8, 16, 17, 40, 64])
def test_bf16_small_m(lib, coracle, m):
    n, k = 256, 320
    w = make_ternary(n, k, 0.40, 50 + m)
    fmt = DeviceFormat(w)
    x = make_bf16_activations(m, k, 60 + m)
    scale = np.array([0.7, 1.9], np.float32)
    got = run_bf16(lib, fmt, x, scale, 2)
    _check_bf16(got, coracle.spmm_bf16(x, w, scale, 2))


def test_bf16_golden_fixture(lib):
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "linear_8x128x192.npz"))
    f = np.load(os.path.join(os.path.dirname(__file__), "golden", "format_128x192.npz"))
    fmt = DeviceFormat(f["w"])
    _check_bf16(run_bf16(lib, fmt, g["x_bf16"], g["scale"], 1), g["ref_fp64"])
    ws_num = int(g["ws_num"])
    assert (run_i8(lib, fmt, g["x_q"], g["s"], g["ws"], ws_num, "bitlinear_TernaSpMM_decode") == g["out_i8_decode"]).all()
    assert (run_i8(lib, fmt, g["x_q"], g["s"], g["ws"], ws_num, "bitlinear_TernaSpMM_prefill") == g["out_i8_prefill"]).all()


def test_bf16_config1(lib):
    """M=8, K=N=2560, P(0)=0.45, one fp32 scale ~ U[0.5, 2]."""
    n = k = 2560
    m = 8
    w = make_ternary(n, k, 0.45, seed_for(1, 0))
    fmt = DeviceFormat(w)
    x = make_bf16_activations(m, k, seed_for(1, 1))
    scale = np.random.default_rng(seed_for(1, 2)).uniform(0.5, 2.0, 1).astype(np.float32)
    got = run_bf16(lib, fmt, x, scale, 1)
    _check_bf16(got, O.spmm_bf16_golden(x, w, scale, 1))


@pytest.mark.parametrize("n,k", [(3840, 2560), (2560, 2560), (13824, 2560), (2560, 6912)])
@pytest.mark.parametrize("m", [1, 8, 16])
def test_bf16_2b_layer_shapes(lib, m, n, k):
    w = make_ternary(n, k, 0.40, seed_for(2, n % 7))
    fmt = DeviceFormat(w)
    x = make_bf16_activations(m, k, seed_for(2, 20 + m))
    scale = np.array([1.37], np.float32)
    got = run_bf16(lib, fmt, x, scale, 1)
    _check_bf16(got, O.spmm_bf16_golden(x, w, scale, 1))


@pytest.mark.parametrize("n,k", [(2560, 2560), (2560, 6912)])
@pytest.mark.parametrize("kind", ["p20", "p33", "p45", "p60", "skewed"])
def test_bf16_sparsity_sweep_m16(lib, n, k, kind):
    seed = seed_for(4, len(kind) + k % 5)
    w = make_row_skewed(n, k, seed) if kind == "skewed" else make_ternary(n, k, int(kind[1:]) / 100.0, seed)
    fmt = DeviceFormat(w)
    x = make_bf16_activations(16, k, seed + 1)
    scale = np.array([0.93], np.float32)
    got = run_bf16(lib, fmt, x, scale, 1)
    _check_bf16(got, O.spmm_bf16_golden(x, w, scale, 1))


def test_bf16_linearity_and_zero_weights(lib):
    """Properties that hold at any size: W == 0 -> output exactly 0; doubling the scale doubles
    every output exactly (power of two); negating x negates the output (to within one bf16 step:
    the matrix cores' internal fp32 summation is not exactly sign-symmetric)."""
    n, k, m = 2560, 2560, 8
    fmt0 = DeviceFormat(np.zeros((n, k), np.int8))
    x = make_bf16_activations(m, k, 71)
    assert not run_bf16(lib, fmt0, x, np.array([1.0], np.float32), 1).any()
    fmt = DeviceFormat(make_ternary(n, k, 0.4, 72))
    a = run_bf16(lib, fmt, x, np.array([0.75], np.float32), 1)
    b = run_bf16(lib, fmt, x, np.array([1.5], np.float32), 1)
    assert (O.bf16_bits_to_f32(b) == 2 * O.bf16_bits_to_f32(a)).all()
    c = run_bf16(lib, fmt, x ^ np.uint16(0x8000), np.array([0.75], np.float32), 1)
    _assert_negation_symmetric(a, c)


def test_call_site_mirror_pads_and_slices(lib, coracle):
    """TernaInfer_linear (the model.py:45-92 mirror): M=3 is padded to 8 rows and sliced back."""
    import ternainfer_amd as T
    n, k, m = 256, 192, 3
    w = make_ternary(n, k, 0.4, 81)
    fmt = DeviceFormat(w)
    xq, s = make_int8_activations(m, k, 82)
    out = T.TernaInfer_linear(torch.from_numpy(xq).cuda(), fmt.vals, fmt.off, fmt.med, fmt.bm,
                              T.get_global_workspace(), torch.from_numpy(s.view(np.int16)).cuda().view(torch.bfloat16),
                              torch.from_numpy(WS.view(np.int16)).cuda().view(torch.bfloat16), 2, n)
    torch.cuda.synchronize()
    assert out.shape == (m, n) and out.dtype == torch.bfloat16
    got = out.view(torch.int16).cpu().numpy().view(np.uint16)
    assert (got == coracle.spmm_i8(xq, w, s, WS, 2, 0)).all()


def test_graph_capture_replays(lib):
    """The entry point only enqueues: capture it in a HIP graph, replay with eager work between."""
    n, k, m = 2560, 2560, 8
    w = make_ternary(n, k, 0.4, 91)
    fmt = DeviceFormat(w)
    x_bits = make_bf16_activations(m, k, 92)
    scale = np.array([1.1], np.float32)
    eager = run_bf16(lib, fmt, x_bits, scale, 1)
    x = torch.from_numpy(x_bits.view(np.int16)).cuda()
    sc = torch.from_numpy(scale).cuda()
    out = torch.zeros((m, n), dtype=torch.int16, device="cuda")
    st = torch.cuda.Stream()
    st.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        with torch.cuda.graph(g, stream=st):
            lib.bitlinear_TernaSpMM_bf16(vp(x), vp(fmt.bm), vp(fmt.off), vp(fmt.med), vp(fmt.vals), vp(out), vp(sc),
                                         1, m, n, k, 1, None, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    for _ in range(3):
        out.fill_(0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert (out.cpu().numpy().view(np.uint16) == eager).all()


# ------------------------------------------------------------------------------- MFMA-tiled (large-M) kernel
@pytest.mark.parametrize("m", [1, 8, 33, 64, 100, 256, 300])
@pytest.mark.parametrize("n,k", [(256, 64), (320, 128), (512, 320)])
def test_bf16_prefill_kernel_small_shapes(lib, coracle, m, n, k):
    """The forced _prefill entry runs the MFMA-tiled kernel at any M: ragged M, N not a multiple
    of the 256-wide tile, one to five k-steps."""
    w = make_ternary(n, k, 0.40, 300 + m + n)
    fmt = DeviceFormat(w)
    x = make_bf16_activations(m, k, 310 + m + k, outlier_frac=0.01)
    scale = np.array([0.7, 1.9], np.float32)
    got = run_bf16(lib, fmt, x, scale, 2, "bitlinear_TernaSpMM_bf16_prefill")
    _check_bf16(got, coracle.spmm_bf16(x, w, scale, 2))


@pytest.mark.parametrize("m", [65, 128, 256, 384])
@pytest.mark.parametrize("n,k,ws_num", [(256, 192, 1), (3840, 128, 3), (640, 320, 2)])
def test_int8_prefill_kernel_bit_exact(lib, m, n, k, ws_num):
    """int8 activations through the bf16 MFMA tiles: every product and partial sum is an integer
    below 2^24, so the result must equal the integer oracle bit for bit."""
    w = make_ternary(n, k, 0.40, 320 + m + n)
    fmt = DeviceFormat(w)
    xq, s = make_int8_activations(m, k, 330 + m + k)
    want = O.spmm_i8(xq, w, s, WS, ws_num, 1)
    got = run_i8(lib, fmt, xq, s, WS, ws_num)                      # M > 64 -> prefill rule; transcode + P2 kernel
    assert (got == want).all()
    got_nw = run_i8(lib, fmt, xq, s, WS, ws_num, workspace=False)  # no workspace -> fused reference-format kernel
    assert (got_nw == want).all()
    got_d = run_i8(lib, fmt, xq, s, WS, ws_num, "bitlinear_TernaSpMM_decode")
    assert (got_d == O.spmm_i8(xq, w, s, WS, ws_num, 0)).all()


def test_prefill_entry_beyond_128_k_steps_falls_back(lib, coracle):
    n, k, m = 64, 64 * 130, 70
    w = make_ternary(n, k, 0.40, 341)
    fmt = DeviceFormat(w)
    x = make_bf16_activations(m, k, 342)
    scale = np.array([1.0], np.float32)
    got = run_bf16(lib, fmt, x, scale, 1, "bitlinear_TernaSpMM_bf16_prefill")
    _check_bf16(got, O.spmm_bf16_golden(x, w, scale, 1))


@pytest.mark.parametrize("n,k", [(3840, 2560), (2560, 2560), (13824, 2560), (2560, 6912)])
@pytest.mark.parametrize("m", [256, 512, 2048])
def test_bf16_prefill_2b_layer_shapes(lib, m, n, k):
    """Prefill shapes with 1% outlier channels (x20).  The fp64 golden is taken on a seeded sample
    of 192 output columns (all rows), which keeps the host matmul small; the whole output is
    also checked for the size-independent property out(-x) == -out(x)."""
    w = make_ternary(n, k, 0.40, seed_for(3, n % 7))
    fmt = DeviceFormat(w)
    x = make_bf16_activations(m, k, seed_for(3, 30 + m % 97), outlier_frac=0.01)
    scale = np.array([1.37], np.float32)
    got = run_bf16(lib, fmt, x, scale, 1)
    cols = np.sort(np.random.default_rng(seed_for(3, 99) + n + 7 * k + m).permutation(n)[:192])
    ref = O.bf16_bits_to_f32(x).astype(np.float64) @ w[cols].astype(np.float64).T * float(scale[0])
    _check_bf16(got[:, cols], ref)
    neg = run_bf16(lib, fmt, x ^ np.uint16(0x8000), scale, 1)
    _assert_negation_symmetric(got, neg)


@pytest.mark.parametrize("n,k,ws_num", [(3840, 2560, 3), (2560, 2560, 1), (13824, 2560, 2), (2560, 6912, 1)])
@pytest.mark.parametrize("m", [256, 512, 2048])
def test_int8_reference_entry_points_2b_layer_shapes_large_m(lib, m, n, k, ws_num):
    """The symbols an unmodified model.py calls (kernels/TernaSpMM.cu:25, :110), on reference-format pointers, at
    the prefill sizes of the four 2B matrices with their weight-scale group counts: with the call site's workspace
    (transcode + P2 kernel), without one (fused reference-format kernel), and the forced _prefill entry.  Bit-exact
    against the integer oracle on a seeded sample of 256 columns that straddles every group boundary; the three
    routes must also agree with each other on the WHOLE output."""
    w = make_ternary(n, k, 0.40, seed_for(3, 40 + n % 7))
    fmt = DeviceFormat(w)
    xq, s = make_int8_activations(m, k, seed_for(3, 50 + m % 97))
    s = s.copy()
    s[m // 3] = 0                                                          # the visitor's s == 0 -> coefficient 0 rule
    rng = np.random.default_rng(seed_for(3, 60 + n % 7 + m % 5))
    edges = [c for b in (2560, 3200, n // 2, n - 1, 0) for c in (b - 1, b, b + 127, b + 128) if 0 <= c < n]
    cols = np.unique(np.concatenate([rng.permutation(n)[:256], np.array(edges)]))
    want = O.spmm_i8(xq, w, s, WS, ws_num, 1, cols=cols)
    a = run_i8(lib, fmt, xq, s, WS, ws_num)                                # M > 64: prefill rule, transcode route
    assert (a[:, cols] == want).all()
    b = run_i8(lib, fmt, xq, s, WS, ws_num, workspace=False)               # fused reference-format kernel
    assert (b == a).all()
    c = run_i8(lib, fmt, xq, s, WS, ws_num, "bitlinear_TernaSpMM_prefill")
    assert (c == a).all()


@pytest.mark.parametrize("n,k", [(3840, 2560), (2560, 2560), (13824, 2560), (2560, 6912)])
def test_packed_bf16_2b_layer_shapes_m512(lib, n, k):
    w = make_ternary(n, k, 0.40, seed_for(3, 70 + n % 7))
    packed = repack(lib, DeviceFormat(w))
    x = make_bf16_activations(512, k, seed_for(3, 71 + n % 7), outlier_frac=0.01)
    scale = np.array([0.83], np.float32)
    got = run_bf16_packed(lib, packed, n, x, scale, 1)
    cols = np.sort(np.random.default_rng(seed_for(3, 72 + n % 7)).permutation(n)[:192])
    ref = O.bf16_bits_to_f32(x).astype(np.float64) @ w[cols].astype(np.float64).T * float(scale[0])
    _check_bf16(got[:, cols], ref)


def _run_packed_ws(lib, act, packed, n, x_or_q, s_bits, scale_or_ws, ws_num, route, work):
    m, k = x_or_q.shape
    out = torch.full((m, n), -1, dtype=torch.int16, device="cuda")
    nbytes = work.numel() if work is not None else 0
    print(f"[case] packed_ws {act} M={m} N={n} K={k} route={route} workspace={nbytes}", flush=True)
    if act == "int8":
        x, sd = torch.from_numpy(x_or_q).cuda(), torch.from_numpy(s_bits.view(np.int16)).cuda()
        wsd = torch.from_numpy(scale_or_ws.view(np.int16)).cuda()
        lib.bitlinear_TernaSpMM_packed_ws(vp(x), vp(packed), vp(out), vp(sd), vp(wsd), ws_num, m, n, k, route,
                                          vp(work) if work is not None else None, nbytes, _stream())
    else:
        x, sc = torch.from_numpy(x_or_q.view(np.int16)).cuda(), torch.from_numpy(scale_or_ws).cuda()
        lib.bitlinear_TernaSpMM_bf16_packed_ws(vp(x), vp(packed), vp(out), vp(sc), ws_num, m, n, k, route,
                                               vp(work) if work is not None else None, nbytes, _stream())
    torch.cuda.synchronize()
    return out.cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("m,n,k,ws_num", [(100, 256, 2048, 2), (128, 128, 6400, 1), (300, 384, 1536, 3),
                                          (256, 2560, 6912, 1), (512, 2560, 6912, 1), (256, 3840, 2560, 3), (192, 2560, 2560, 1)])
def test_packed_split_k_with_workspace(lib, m, n, k, ws_num):
    """Few output tiles for the chip + scratch memory: the K steps are spread over several workgroups per tile and a
    second launch sums the partial planes in split order.  int8: bit-exact against the integer oracle (and hence
    identical to the unsplit call); bf16: within the family's tolerance.  A workspace too small for one plane, or
    none, must fall back to the single launch."""
    w = make_ternary(n, k, 0.40, 460 + m + n % 97)
    packed = repack(lib, DeviceFormat(w))
    work = torch.full((8 * m * n * 4 + 64,), 0x55, dtype=torch.int8, device="cuda")[16:]     # 16-byte aligned, poisoned
    cols = np.sort(np.random.default_rng(461 + m + n).permutation(n)[:256]) if n > 256 else np.arange(n)
    xq, s = make_int8_activations(m, k, 462 + m)
    s = s.copy()
    s[m // 2] = 0
    want = O.spmm_i8(xq, w, s, WS, ws_num, 1, cols=cols)
    split = _run_packed_ws(lib, "int8", packed, n, xq, s, WS, ws_num, 8, work)          # MFMA kernel, reference's rule by M
    assert (split[:, cols] == want).all()
    plain = _run_packed_ws(lib, "int8", packed, n, xq, s, WS, ws_num, 8, None)
    assert (plain == split).all()
    tiny = _run_packed_ws(lib, "int8", packed, n, xq, s, WS, ws_num, 8, work[:m * n * 4 - 16])
    assert (tiny == split).all()
    x = make_bf16_activations(m, k, 463 + m, outlier_frac=0.01)
    scale = np.array([0.7, 1.9, 1.3], np.float32)
    ref = O.bf16_bits_to_f32(x).astype(np.float64) @ w[cols].astype(np.float64).T * \
        scale[O.ws_group_decode(cols, n, ws_num)].astype(np.float64)[None, :]
    _check_bf16(_run_packed_ws(lib, "bf16", packed, n, x, None, scale, ws_num, 1, work)[:, cols], ref)
    _check_bf16(_run_packed_ws(lib, "bf16", packed, n, x, None, scale, ws_num, 1, None)[:, cols], ref)


@pytest.mark.parametrize("with_ws", [False, True])
@pytest.mark.parametrize("m", [32, 33, 48, 64, 65, 96, 128, 129, 192, 193, 256, 257])
@pytest.mark.parametrize("n,k,ws_num", [(8256, 192, 1), (3840, 128, 3), (2560, 128, 1), (256, 4160, 2)])
def test_packed_kernel_choice_boundaries(lib, m, n, k, ws_num, with_ws):
    """The library picks the small-M or the MFMA-tiled kernel by shape (more than 512 bands: up to 32 rows; long K,
    int8, 160 bands or fewer, scratch at hand: other cuts); whatever it picks, int8 results follow the reference's M <= 64 epilogue rule
    bit for bit and bf16 results stay within tolerance, on both sides of every cut."""
    w = make_ternary(n, k, 0.40, 470 + n % 89)
    packed = repack(lib, DeviceFormat(w))
    work = torch.empty(8 * m * n * 4, dtype=torch.int8, device="cuda") if with_ws else None
    xq, s = make_int8_activations(m, k, 471 + m)
    cols = np.sort(np.random.default_rng(472 + n).permutation(n)[:512])
    got = _run_packed_ws(lib, "int8", packed, n, xq, s, WS, ws_num, 0, work)
    assert (got[:, cols] == O.spmm_i8(xq, w, s, WS, ws_num, 0 if m <= 64 else 1, cols=cols)).all()
    x = make_bf16_activations(m, k, 473 + m)
    scale = np.array([0.7, 1.9, 1.3], np.float32)
    ref = O.bf16_bits_to_f32(x).astype(np.float64) @ w[cols].astype(np.float64).T * \
        scale[O.ws_group_decode(cols, n, ws_num)].astype(np.float64)[None, :]
    _check_bf16(_run_packed_ws(lib, "bf16", packed, n, x, None, scale, ws_num, 0, work)[:, cols], ref)


def _random_shapes(count, seed):
    """Seeded shapes off the beaten track: N and K any multiple of 64 (N up to 1536: 96 bands, K up to 40 k-tiles), M on
    both sides of every kernel cut, one to four weight-scale groups."""
    rng = np.random.default_rng(seed)
    shapes = []
    for i in range(count):
        n = 64 * int(rng.integers(1, 25))
        k = 64 * int(rng.integers(1, 41))
        m = int(rng.choice([rng.integers(1, 17), rng.integers(17, 65), rng.integers(65, 200), rng.integers(200, 420)]))
        ws_num = int(rng.choice([g for g in (1, 2, 3, 4) if n % g == 0]))          # groups that divide N, as every caller's do
        shapes.append((m, n, k, ws_num, float(rng.choice([0.2, 0.4, 0.6])), 9000 + i))
    return shapes


@pytest.mark.parametrize("m,n,k,ws_num,p0,seed", _random_shapes(24, 20260900))
def test_random_shapes_int8_bit_exact_on_every_route(lib, m, n, k, ws_num, p0, seed):
    """Shapes nobody tuned for, through the reference's entry point (with and without its workspace) and through the P2
    entry points (default route with and without scratch, both forced kernels): the integers of every route are the
    oracle's, bit for bit, under the epilogue rule that route follows."""
    w = make_ternary(n, k, p0, seed)
    fmt = DeviceFormat(w)
    xq, s = make_int8_activations(m, k, seed + 1)
    if m > 2:
        s = s.copy()
        s[m // 3] = 0                                                    # a row whose scale is zero
    by_m = O.spmm_i8(xq, w, s, WS, ws_num, 0 if m <= 64 else 1)
    for workspace in (True, False):
        assert (run_i8(lib, fmt, xq, s, WS, ws_num, workspace=workspace) == by_m).all(), f"reference entry point, workspace={workspace}"
    packed = repack(lib, fmt)
    work = torch.empty(8 * m * n * 4, dtype=torch.int8, device="cuda")
    assert (_run_packed_ws(lib, "int8", packed, n, xq, s, WS, ws_num, 0, None) == by_m).all(), "P2, default route"
    assert (_run_packed_ws(lib, "int8", packed, n, xq, s, WS, ws_num, 0, work) == by_m).all(), "P2, default route, scratch"
    assert (run_i8_packed(lib, packed, n, xq, s, WS, ws_num, 1) == O.spmm_i8(xq, w, s, WS, ws_num, 1)).all(), "P2, MFMA-tiled kernel"
    if m <= 64:
        assert (run_i8_packed(lib, packed, n, xq, s, WS, ws_num, 2) == by_m).all(), "P2, small-M kernel"


# ------------------------------------------------------------------------------- P2 layout (load-time repack)
@pytest.mark.parametrize("kind", ["iid40", "skewed", "dense", "empty", "sparse97"])
def test_repack_is_bit_exact(lib, kind):
    """repack(encode(W)) == pack(W): the device transcoder against the oracle's packing of the
    original matrix, and unpack(pack(W)) == W closes the round trip."""
    n, k = 256, 320
    w = {"iid40": lambda: make_ternary(n, k, 0.40, 1), "skewed": lambda: make_row_skewed(n, k, 3),
         "dense": lambda: make_ternary(n, k, 0.0, 4), "empty": lambda: np.zeros((n, k), np.int8),
         "sparse97": lambda: make_ternary(n, k, 0.97, 5)}[kind]()
    got = repack(lib, DeviceFormat(w)).cpu().numpy().view(np.uint32)
    assert (got == O.pack_p2(w).reshape(-1)).all()
    assert (O.unpack_p2(got, n, k) == w).all()


@pytest.mark.parametrize("n,k", [(13824, 2560), (2560, 6912)])
def test_repack_full_size_round_trip(lib, n, k):
    w = make_ternary(n, k, 0.40, seed_for(2, 50 + n % 7))
    got = repack(lib, DeviceFormat(w)).cpu().numpy().view(np.uint32)
    assert (O.unpack_p2(got, n, k) == w).all()


@pytest.mark.parametrize("m", [1, 8, 16, 24, 64, 65, 128, 300])
@pytest.mark.parametrize("n,k,ws_num", [(256, 192, 1), (640, 320, 2), (3840, 128, 3)])
def test_packed_int8_bit_exact(lib, m, n, k, ws_num):
    w = make_ternary(n, k, 0.40, 400 + m + n)
    packed = repack(lib, DeviceFormat(w))
    xq, s = make_int8_activations(m, k, 410 + m + k)
    mode = 0 if m <= 64 else 1
    assert (run_i8_packed(lib, packed, n, xq, s, WS, ws_num) == O.spmm_i8(xq, w, s, WS, ws_num, mode)).all()
    assert (run_i8_packed(lib, packed, n, xq, s, WS, ws_num, 2) == O.spmm_i8(xq, w, s, WS, ws_num, 0)).all()
    assert (run_i8_packed(lib, packed, n, xq, s, WS, ws_num, 1) == O.spmm_i8(xq, w, s, WS, ws_num, 1)).all()


@pytest.mark.parametrize("m", [1, 8, 16])
@pytest.mark.parametrize("n,k,ws_num", [(13824, 2560, 2), (8256, 192, 1), (8320, 64, 4)])
def test_packed_int8_many_bands_bit_exact(lib, m, n, k, ws_num):
    """More than 512 bands: the small-M kernel takes two bands per workgroup (gate+up and two synthetic
    shapes with 516 / 520 bands, one to three k-tiles, several weight-scale groups)."""
    w = make_ternary(n, k, 0.40, 430 + m + n % 97)
    packed = repack(lib, DeviceFormat(w))
    xq, s = make_int8_activations(m, k, 431 + m + k)
    print(f"[case] packed int8, many bands m={m} n={n} k={k}", flush=True)
    assert (run_i8_packed(lib, packed, n, xq, s, WS, ws_num) == O.spmm_i8(xq, w, s, WS, ws_num, 0)).all()


@pytest.mark.parametrize("m", [1, 70, 256])
@pytest.mark.parametrize("n,k,ws_num", [(64, 64, 1), (192, 448, 1), (3840, 2560, 3), (2560, 6912, 1)])
def test_packed_int8_mfma_kernel_tile_counts_and_2b_shapes(lib, m, n, k, ws_num):
    """The large-M int8 kernel walks K two 64-column tiles at a time: one tile (K = 64), an odd count
    (K = 448), and the even counts of the 2B matrices, forced onto that kernel at every M."""
    w = make_ternary(n, k, 0.40, 440 + m + n)
    packed = repack(lib, DeviceFormat(w))
    xq, s = make_int8_activations(m, k, 450 + m + k)
    assert (run_i8_packed(lib, packed, n, xq, s, WS, ws_num, 1) == O.spmm_i8(xq, w, s, WS, ws_num, 1)).all()


@pytest.mark.parametrize("route", [1, 2])
@pytest.mark.parametrize("m", [1, 3, 16, 17, 64, 100, 256, 300])
@pytest.mark.parametrize("n,k", [(256, 64), (320, 128), (512, 320)])
def test_packed_bf16_both_kernels(lib, coracle, route, m, n, k):
    """route 1 = MFMA-tiled kernel, route 2 = small-M kernel, each at every M."""
    w = make_ternary(n, k, 0.40, 420 + m + n)
    packed = repack(lib, DeviceFormat(w))
    x = make_bf16_activations(m, k, 430 + m + k, outlier_frac=0.01)
    scale = np.array([0.7, 1.9], np.float32)
    _check_bf16(run_bf16_packed(lib, packed, n, x, scale, 2, route), coracle.spmm_bf16(x, w, scale, 2))


@pytest.mark.parametrize("n,k", [(3840, 2560), (2560, 2560), (13824, 2560), (2560, 6912)])
@pytest.mark.parametrize("m", [1, 8, 16, 256, 2048])
def test_packed_bf16_2b_layer_shapes(lib, m, n, k):
    w = make_ternary(n, k, 0.40, seed_for(2, n % 7))
    packed = repack(lib, DeviceFormat(w))
    x = make_bf16_activations(m, k, seed_for(2, 60 + m % 97), outlier_frac=0.01 if m >= 256 else 0.0)
    scale = np.array([1.37], np.float32)
    got = run_bf16_packed(lib, packed, n, x, scale, 1)
    cols = np.sort(np.random.default_rng(seed_for(2, 98)).permutation(n)[:192]) if m >= 256 else np.arange(n)
    ref = O.bf16_bits_to_f32(x).astype(np.float64) @ w[cols].astype(np.float64).T * float(scale[0])
    _check_bf16(got[:, cols], ref)


@pytest.mark.parametrize("m,with_ws", [(2560, False), (2560, True), (300, True)])
def test_packed_bf16_scale_groups_inside_a_tile_at_large_m(lib, m, with_ws):
    """Four weight-scale groups of 1072 features: the boundaries fall in the middle of a 32-feature tile, so every
    column takes its own scale.  Only the 128 x 64 tile of the MFMA kernel carries that epilogue; a call the planner would
    give 256-wide tiles (M = 2560: 680 of them) or split-K planes (M = 300 with scratch) must end up there too."""
    n, k, ws_num = 4288, 128, 4
    w = make_ternary(n, k, 0.40, 480 + m)
    packed = repack(lib, DeviceFormat(w))
    x = make_bf16_activations(m, k, 481 + m)
    scale = np.array([0.7, 1.9, 1.3, 0.45], np.float32)
    work = torch.empty(8 * m * n * 4, dtype=torch.int8, device="cuda") if with_ws else None
    got = _run_packed_ws(lib, "bf16", packed, n, x, None, scale, ws_num, 1, work)
    near = np.concatenate([np.arange(b - 40, b + 40) for b in (1072, 2144, 3216)])
    cols = np.unique(np.concatenate([near, np.random.default_rng(482).permutation(n)[:128], [0, n - 1]]))
    ref = O.bf16_bits_to_f32(x).astype(np.float64) @ w[cols].astype(np.float64).T * \
        scale[O.ws_group_decode(cols, n, ws_num)].astype(np.float64)[None, :]
    _check_bf16(got[:, cols], ref)


def test_large_m_with_workspace_matches_without(lib):
    """The transcode-into-workspace route and the fused route compute the same sums in a different
    order; both must sit within tolerance of the golden, and the int8 family must agree bit for bit."""
    n, k, m = 512, 640, 200
    w = make_ternary(n, k, 0.40, 441)
    fmt = DeviceFormat(w)
    x = make_bf16_activations(m, k, 442, outlier_frac=0.01)
    scale = np.array([1.0], np.float32)
    ref = O.spmm_bf16_golden(x, w, scale, 1)
    _check_bf16(run_bf16(lib, fmt, x, scale, 1, workspace=True), ref)
    _check_bf16(run_bf16(lib, fmt, x, scale, 1, workspace=False), ref)


@pytest.mark.parametrize("n", [384, 192])
def test_large_m_output_store_paths_agree(lib, n):
    """The MFMA-tiled kernels write whole rows (16 bytes per lane, through an LDS tile) when the output pointer
    and row pitch are multiples of 16 bytes and 8-byte pieces otherwise: an output buffer shifted by 8 bytes must
    receive the same bits, for both families, with ragged M and a feature count that leaves the last tile partly
    outside N, and nothing outside the [M][N] block may be written."""
    k, m = 320, 200
    w = make_ternary(n, k, 0.40, 461 + n)
    packed = repack(lib, DeviceFormat(w))
    x = make_bf16_activations(m, k, 462, outlier_frac=0.01)
    xq, s = make_int8_activations(m, k, 463)
    scale = np.array([1.25], np.float32)
    want_bf = run_bf16_packed(lib, packed, n, x, scale, 1, route=1)
    want_i8 = run_i8_packed(lib, packed, n, xq, s, WS, 1, route=9)     # MFMA-tiled kernel, prefill epilogue
    xd = torch.from_numpy(x.view(np.int16)).cuda()
    xqd = torch.from_numpy(xq).cuda()
    sd = torch.from_numpy(s.view(np.int16)).cuda()
    wsd = torch.from_numpy(WS.view(np.int16)).cuda()
    scd = torch.from_numpy(scale).cuda()
    for shift in (4, 8):       # elements: 8 bytes (pieces), 16 bytes (rows again)
        buf = torch.full((m * n + 64,), -1, dtype=torch.int16, device="cuda")
        out = buf[shift:shift + m * n]
        print(f"[case] bitlinear_TernaSpMM_bf16_packed M={m} N={n} K={k}, output shifted by {2 * shift} bytes", flush=True)
        lib.bitlinear_TernaSpMM_bf16_packed(vp(xd), vp(packed), vp(out), vp(scd), 1, m, n, k, 1, _stream())
        torch.cuda.synchronize()
        got = buf.cpu().numpy().view(np.uint16)
        assert (got[shift:shift + m * n].reshape(m, n) == want_bf).all()
        assert (got[:shift] == 0xFFFF).all() and (got[shift + m * n:] == 0xFFFF).all()
        buf.fill_(-1)
        print(f"[case] bitlinear_TernaSpMM_packed M={m} N={n} K={k}, output shifted by {2 * shift} bytes", flush=True)
        lib.bitlinear_TernaSpMM_packed(vp(xqd), vp(packed), vp(out), vp(sd), vp(wsd), 1, m, n, k, 9, _stream())
        torch.cuda.synchronize()
        got = buf.cpu().numpy().view(np.uint16)
        assert (got[shift:shift + m * n].reshape(m, n) == want_i8).all()
        assert (got[:shift] == 0xFFFF).all() and (got[shift + m * n:] == 0xFFFF).all()


def test_spbitlinear_module_reference_and_repacked_agree(lib, coracle):
    """The call-site mirror: SpBitLinear from a reference-format checkpoint dict, with and without
    the load-time repack, against the oracle on the module's own quantised activations."""
    import ternainfer_amd as T
    n, k, m = 384, 256, 5
    w = make_ternary(n, k, 0.4, 451)
    vals, off, med, bm = T.compress_weight(torch.from_numpy(w))
    ws = torch.tensor([1.59375, 0.8125, 0.0, 0.0], dtype=torch.bfloat16)
    dic = {"l.weight_compressed_val": vals, "l.weight_TileOffsets_global": off, "l.weight_TileOffsets_median": med,
           "l.weight_bitmap": bm, "l.weight_scale": ws}
    x = torch.from_numpy(O.bf16_bits_to_f32(make_bf16_activations(m, k, 452))).to(torch.bfloat16).cuda()
    print("[case] SpBitLinear reference-format vs repacked", flush=True)
    a = T.SpBitLinear(k, n, dic, "l")(x)
    b = T.SpBitLinear(k, n, dic, "l", repack=True)(x)
    torch.cuda.synchronize()
    assert a.shape == (m, n) and torch.equal(a, b)
    xq, s = T.SpBitLinear(k, n, dic, "l").quant_input(x)
    want = coracle.spmm_i8(xq.cpu().numpy(), w, s.to(torch.bfloat16).view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1),
                           ws.view(torch.int16).numpy().view(np.uint16), 2, 0)
    assert (a.view(torch.int16).cpu().numpy().view(np.uint16) == want).all()


def test_kernel_binary_reference_command_line():
    """tests/test_kernel (HIP build of the reference's micro-test, same CLI): the documented
    invocation `8 2560 2560 45 7` must agree exactly with the dense bf16 GEMM (x == 1 makes every
    output an integer row sum), for both families and the repacked layout."""
    import subprocess
    exe = os.path.join(os.path.dirname(__file__), "test_kernel")
    if not os.path.exists(exe):
        pytest.fail("tests/test_kernel is not built: run `bash kernels/compile.sh`")
    print("[case] tests/test_kernel 8 2560 2560 45 7", flush=True)
    r = subprocess.run([exe, "8", "2560", "2560", "45", "7"], capture_output=True, text=True, timeout=120)
    print(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("TotalError: 0.00") == 4


@pytest.mark.parametrize("env", [{"TERNASPMM_PREFILL_DMA": "0"},
                                 {"TERNASPMM_PREFILL_DMA": "0", "TERNASPMM_PREFILL_BM": "128"},
                                 {"TERNASPMM_PREFILL_BM": "128", "TERNASPMM_PREFILL_BN": "256"},
                                 {"TERNASPMM_PREFILL_BM": "128", "TERNASPMM_PREFILL_BN": "128"},
                                 {"TERNASPMM_PREFILL_BN": "256"}, {"TERNASPMM_PREFILL_BN": "128"},
                                 {"TERNASPMM_PREFILL_BM": "256"}, {"TERNASPMM_PREFILL_BM": "96"},
                                 {"TERNASPMM_PREFILL_XCD_MAP": "1"}, {"TERNASPMM_PREFILL_XCD_MAP": "1", "TERNASPMM_PREFILL_BM": "128"},
                                 {"TERNASPMM_DECODE_WAVES": "4"}, {"TERNASPMM_DECODE_WAVES": "8"}, {"TERNASPMM_DECODE_WAVES": "16"},
                                 {"TERNASPMM_DECODE_BANDS": "1"}, {"TERNASPMM_FUSED_BANDS": "1"},
                                 {"TERNASPMM_FUSED_BANDS_WAVES": "16"}, {"TERNASPMM_FUSED_WAVES": "8"}, {"TERNASPMM_FUSED_WAVES": "16"},
                                 {"TERNASPMM_ATTN_WAVES": "4"}, {"TERNASPMM_ATTN_SPLITS": "2"}, {"TERNASPMM_ATTN_SPLITS": "8"},
                                 {"TERNASPMM_ATTN_XCD_GROUPS": "0"}, {"TERNASPMM_PREFILL_SPLITS": "1"},
                                 {"TERNASPMM_PREFILL_SPLITS": "5"}])
def test_tile_and_path_overrides(env):
    """Every tile shape, launch shape and path behind the library's tuning overrides
    (read once per process, hence a child process): tests/env_variant_check.py must pass under each."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    print(f"[case] override {env}", flush=True)
    r = subprocess.run([sys.executable, "-u", "-m", "tests.env_variant_check"], cwd=root,
                       env={**os.environ, "TERNASPMM_TUNING": "1", **env},
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "override check ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


def test_repack_cache_behind_reference_entry_points():
    """TERNASPMM_REPACK_CACHE=1 (read once per process, hence a child process): tests/repack_cache_check.py."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-u", "-m", "tests.repack_cache_check"], cwd=root,
                       env={**os.environ, "TERNASPMM_REPACK_CACHE": "1"}, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "repack cache check ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
    # a weight rewritten under the same pointers without ternaspmm_repack_cache_clear(): the launch that follows reports
    # the stale copy, the next call drops it with a warning and serves the new weight correctly ...
    r = subprocess.run([sys.executable, "-u", "-m", "tests.repack_cache_check", "stale"], cwd=root,
                       env={**os.environ, "TERNASPMM_REPACK_CACHE": "1"}, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "stale copy dropped and rebuilt ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
    assert "no longer matched the tensors it was made from" in r.stdout and "Warning" in r.stdout
    # ... or, with TERNASPMM_REPACK_CACHE_STRICT=1, ends the process as every error of the library does
    r = subprocess.run([sys.executable, "-u", "-m", "tests.repack_cache_check", "stale"], cwd=root,
                       env={**os.environ, "TERNASPMM_REPACK_CACHE": "1", "TERNASPMM_REPACK_CACHE_STRICT": "1"},
                       capture_output=True, text=True, timeout=300)
    assert r.returncode != 0 and "no longer matched the tensors it was made from" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
    assert "stale copy dropped" not in r.stdout
    # the byte limit: least recently used copies go, a weight that does not fit is served without a copy
    r = subprocess.run([sys.executable, "-u", "-m", "tests.repack_cache_check", "limit"], cwd=root,
                       env={**os.environ, "TERNASPMM_REPACK_CACHE": "1"}, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "cache limit check ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


def test_benchmark_entry_point_times_and_leaves_the_result(lib, capfd):
    """bitlinear_TernaSpMM_benchmark(mode, warmup, iters, <the 15 arguments>) (kernels/TernaSpMM.cu:141-236):
    runs the chosen path, prints one 'Shape(M=.., N=.., K=..): <t> us' line, and `out` holds the result."""
    import re
    n, k = 256, 192
    w = make_ternary(n, k, 0.40, 980)
    fmt = DeviceFormat(w)
    for mode, m, ep_mode in [(0, 8, 0), (2, 8, 0), (1, 8, 1), (0, 100, 1), (2, 100, 0)]:
        xq, s = make_int8_activations(m, k, 981 + m)
        x, sd = torch.from_numpy(xq).cuda(), torch.from_numpy(s.view(np.int16)).cuda()
        ws = torch.from_numpy(WS.view(np.int16)).cuda()
        out = torch.full((m, n), -1, dtype=torch.int16, device="cuda")
        work = _workspace(m, n, k)
        print(f"[case] benchmark entry mode={mode} M={m}", flush=True)
        capfd.readouterr()
        lib.bitlinear_TernaSpMM_benchmark(mode, 2, 5, vp(x), vp(fmt.bm), vp(fmt.off), vp(fmt.med), vp(fmt.vals), vp(out),
                                          vp(sd), vp(ws), 2, m, n, k, 7, vp(work), _stream())
        torch.cuda.synchronize()
        text = capfd.readouterr().out
        match = re.search(r"Shape\(M=(\d+), N=(\d+), K=(\d+)\): ([0-9.]+) us", text)
        assert match, text
        assert (int(match.group(1)), int(match.group(2)), int(match.group(3))) == (m, n, k)
        assert 0.0 < float(match.group(4)) < 1e4
        assert (out.cpu().numpy().view(np.uint16) == O.spmm_i8(xq, w, s, WS, 2, ep_mode)).all()


def test_gpu_sleep_and_error_check(lib):
    """gpu_sleep(us, stream) (kernels/TernaSpMM.cu:454) occupies the stream for about that long;
    checkLastCudaError(line) returns quietly when nothing went wrong."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    lib.gpu_sleep(ctypes.c_double(100.0), _stream())             # warm-up: code object load
    torch.cuda.synchronize()
    e0.record()
    lib.gpu_sleep(ctypes.c_double(3000.0), _stream())
    e1.record()
    torch.cuda.synchronize()
    assert 2.5 <= e0.elapsed_time(e1) <= 30.0
    lib.checkLastCudaError(123)
