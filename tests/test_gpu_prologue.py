"""GPU tests of the fused prologue kernels (residual add / gate -> RMSNorm -> int8 quantisation)
through the C ABI, against the CPU oracle.

Bars: the residual stream and the int8 quantisation are bit-exact (their arithmetic is fully
defined); the norm output is within one bf16 step of the float64 evaluation, the tolerance a
parallel fp32 sum of squares leaves (RMSNorm parity is unpinned: xformers is absent)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import terna_oracle as O
from tests._util import make_bf16_activations

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    from ternainfer_amd import _lib
    return _lib.load()


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16) if a.dtype == np.uint16 else np.ascontiguousarray(a)).cuda()


def _vp(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _run(lib, x, w, eps, residual=None, glu=False, want_y=True, want_q=True):
    m = x.shape[0]
    k = x.shape[1] // 2 if glu else x.shape[1]
    xd, wd = _dev(x), _dev(w)
    rd = _dev(residual) if residual is not None else None
    hd = torch.zeros((m, k), dtype=torch.int16, device="cuda") if residual is not None else None
    yd = torch.zeros((m, k), dtype=torch.int16, device="cuda") if want_y else None
    qd = torch.zeros((m, k), dtype=torch.int8, device="cuda") if want_q else None
    sd = torch.zeros(m, dtype=torch.int16, device="cuda") if want_q else None
    if glu:
        lib.ternaspmm_relu2_mul_rmsnorm_quant(_vp(xd), _vp(wd), eps, _vp(yd), _vp(qd), _vp(sd), m, k, None)
    else:
        lib.ternaspmm_rmsnorm_quant(_vp(xd), _vp(rd), _vp(hd), _vp(wd), eps, _vp(yd), _vp(qd), _vp(sd), m, k, None)
    torch.cuda.synchronize()
    get = lambda t, dt: None if t is None else t.cpu().numpy().view(dt)
    return get(hd, np.uint16), get(yd, np.uint16), get(qd, np.int8), get(sd, np.uint16)


def _assert_within_one_bf16_step(got_bits, want_bits):
    """Monotone integer image of bf16 storage: adjacent values differ by 1."""
    def key(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    d = np.abs(key(got_bits) - key(want_bits))
    assert d.max() <= 1, f"max distance {d.max()} bf16 steps"
    assert (d != 0).mean() < 0.02, f"{(d != 0).mean():.4f} of the outputs are one step off"


def _weight(k, seed):
    return O.f32_to_bf16_bits(np.random.default_rng(seed).uniform(0.5, 1.5, k).astype(np.float32))


@pytest.mark.parametrize("m", [1, 8, 37, 256])
@pytest.mark.parametrize("k", [64, 2560, 6912, 8192])
def test_rmsnorm_quant_plain(lib, m, k):
    x = make_bf16_activations(m, k, 600 + m + k, outlier_frac=0.01)
    w = _weight(k, 601 + k)
    _, y, q, s = _run(lib, x, w, 1e-5)
    _assert_within_one_bf16_step(y, O.rmsnorm(x, w, 1e-5))
    want_q, want_s = O.quant_input(y)                         # the quantiser, on the kernel's own norm output
    assert (s == want_s).all() and (q == want_q).all()


@pytest.mark.parametrize("m,k", [(8, 2560), (300, 2560), (5, 640)])
def test_rmsnorm_quant_with_residual(lib, m, k):
    x = make_bf16_activations(m, k, 610 + m)
    r = make_bf16_activations(m, k, 611 + m, outlier_frac=0.01)
    w = _weight(k, 612)
    h, y, q, s = _run(lib, x, w, 1e-5, residual=r)
    want_h = O.residual_add(x, r)
    assert (h == want_h).all()
    _assert_within_one_bf16_step(y, O.rmsnorm(want_h, w, 1e-5))
    want_q, want_s = O.quant_input(y)
    assert (s == want_s).all() and (q == want_q).all()


@pytest.mark.parametrize("m,f", [(1, 6912), (8, 6912), (100, 6912), (16, 64)])
def test_relu2_mul_rmsnorm_quant(lib, m, f):
    x13 = make_bf16_activations(m, 2 * f, 620 + m + f, outlier_frac=0.01)
    w = _weight(f, 621)
    _, y, q, s = _run(lib, x13, w, 1e-5, glu=True)
    _assert_within_one_bf16_step(y, O.rmsnorm(O.relu2_mul(x13), w, 1e-5))
    want_q, want_s = O.quant_input(y)
    assert (s == want_s).all() and (q == want_q).all()


def test_optional_outputs_do_not_change_the_others(lib):
    x = make_bf16_activations(9, 2560, 630)
    w = _weight(2560, 631)
    _, y, q, s = _run(lib, x, w, 1e-5)
    _, y2, _, _ = _run(lib, x, w, 1e-5, want_q=False)
    _, _, q2, s2 = _run(lib, x, w, 1e-5, want_y=False)
    assert (y == y2).all() and (q == q2).all() and (s == s2).all()


def test_zero_row_quantises_to_zero_with_the_clamped_scale(lib):
    """max|y| = 0 -> s = bf16(127 / 1e-5), q = 0 (model.py:121's clamp_(min=1e-5))."""
    x = np.zeros((2, 128), np.uint16)
    _, y, q, s = _run(lib, x, _weight(128, 640), 1e-5)
    assert (y & 0x7FFF == 0).all() and (q == 0).all()
    assert (s == O.f32_to_bf16_bits(np.array([127.0 / 1e-5], np.float32))[0]).all()


def test_python_wrappers_feed_the_linear(lib):
    """rmsnorm_quant -> TernaInfer_linear_packed equals the unfused sequence on the same inputs."""
    import ternainfer_amd as T
    from tests._util import make_ternary
    n, k, m = 256, 320, 8
    w = make_ternary(n, k, 0.4, 650)
    vals, off, med, bm = [t.cuda() for t in T.compress_weight(torch.from_numpy(w))]
    packed = T.repack_weight(vals, off, med, bm, n, k)
    x = make_bf16_activations(m, k, 651)
    g = _weight(k, 652)
    xt = torch.from_numpy(x.view(np.int16)).cuda().view(torch.bfloat16)
    gt = torch.from_numpy(g.view(np.int16)).cuda().view(torch.bfloat16)
    ws = torch.tensor([1.25, 0, 0, 0], dtype=torch.bfloat16, device="cuda")
    xq, s, h = T.rmsnorm_quant(xt, gt, 1e-5)
    out = T.TernaInfer_linear_packed(xq, packed, s, ws, 1, n)
    y, _ = T.rmsnorm_quant(xt, gt, 1e-5, quant=False)
    yq, ys = O.quant_input(y.view(torch.int16).cpu().numpy().view(np.uint16))
    assert (xq.cpu().numpy() == yq).all()
    want = O.spmm_i8(yq, w, ys, O.f32_to_bf16_bits(np.array([1.25, 0, 0, 0], np.float32)), 1, 0)
    assert (out.view(torch.int16).cpu().numpy().view(np.uint16) == want).all()


@pytest.mark.parametrize("b,v", [(1, 128256), (8, 128256), (3, 1000), (2, 1003), (1, 5), (4, 8192)])
def test_argmax_rows(lib, b, v):
    import ternainfer_amd as T
    """First index of the row maximum, also with ties, -inf entries, NaNs and rows that are not
    16-byte aligned (V % 8 != 0)."""
    rng = np.random.default_rng(900 + v + b)
    x = O.f32_to_bf16_bits(rng.standard_normal((b, v)).astype(np.float32))       # bf16 rounding makes ties common
    xf = O.bf16_bits_to_f32(x)
    if v >= 1000:
        xf[0, 17] = xf[0, 900] = 9.0                                             # a tie: the lower index wins
        xf[-1, 3] = -np.inf
        xf[-1, 11] = np.nan                                                      # never selected
        x = O.f32_to_bf16_bits(xf)
        xf = O.bf16_bits_to_f32(x)
    want = np.array([int(np.flatnonzero(r == np.nanmax(r))[0]) for r in xf], np.int64)
    xd = _dev(x)
    od = torch.full((b,), -1, dtype=torch.int64, device="cuda")
    print(f"[case] argmax b={b} v={v}", flush=True)
    lib.ternaspmm_argmax_bf16(_vp(xd), _vp(od), b, v, None)
    torch.cuda.synchronize()
    assert (od.cpu().numpy() == want).all()
    got = T.argmax_rows(xd.view(torch.bfloat16))
    assert got.shape == (b, 1) and (got.cpu().numpy().ravel() == want).all()


@pytest.mark.parametrize("m,v,k", [(1, 128256, 2560), (8, 128256, 2560), (16, 4096, 2560), (3, 1003, 64), (2, 50, 32),
                                   (5, 8200, 6912), (16, 640, 4128), (3, 1003, 384), (4, 8200, 6912), (1, 50, 128),
                                   (4, 128256, 2560), (2, 4098, 2176), (7, 1003, 192), (6, 4098, 2176), (5, 50, 64)])
def test_lm_head_against_fp64(lib, m, v, k):
    """bf16 LM head: within the bf16 GEMM bar of the fp64 product (max|err| <= 1e-2 max|ref|, median <= 1 ULP
    of the bf16 result), also for V not a multiple of 16 or 4, K that is not a multiple of the unrolled
    depth, and K whose 16 activation rows need more than 64 KB of LDS.  Up to four rows with K a multiple of 128
    take the kernel whose quads of lanes load 64 contiguous bytes, five to eight rows with K a multiple of 64 its form on
    the 32 x 32 MFMA, everything else the plain one."""
    import ternainfer_amd as T
    rng = np.random.default_rng(4100 + m + v + k)
    x = O.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    w = O.f32_to_bf16_bits((rng.standard_normal((v, k)) * 0.05).astype(np.float32))
    ref = O.bf16_bits_to_f32(x).astype(np.float64) @ O.bf16_bits_to_f32(w).astype(np.float64).T
    xd, wd = _dev(x), _dev(w)
    od = torch.zeros((m, v + 8), dtype=torch.int16, device="cuda").view(-1)[: m * v].view(m, v)   # tail stays zero
    print(f"[case] lm_head m={m} v={v} k={k}", flush=True)
    lib.ternaspmm_lm_head_bf16(_vp(xd), _vp(wd), _vp(od), m, v, k, None)
    torch.cuda.synchronize()
    got = O.bf16_bits_to_f32(od.cpu().numpy().view(np.uint16)).astype(np.float64)
    err = np.abs(got - ref)
    assert err.max() <= 1e-2 * np.abs(ref).max()
    ulp = np.maximum(np.abs(ref), 2.0 ** -126) * 2.0 ** -7
    assert np.median(err / ulp) <= 1.0
    got2 = T.lm_head(xd.view(torch.bfloat16), wd.view(torch.bfloat16))
    assert torch.equal(got2.view(torch.int16), od)


# ------------------------------------------------------------------ attention-side kernels
@pytest.mark.parametrize("adjacent", [0, 1])
@pytest.mark.parametrize("b,t,h,kv,d,s_max", [(1, 1, 20, 5, 128, 64), (2, 24, 4, 2, 64, 32), (3, 5, 20, 5, 128, 40),
                                              (2, 3, 4, 2, 24, 16)])
def test_rope_kv_store(lib, b, t, h, kv, d, s_max, adjacent):
    rope = O.rope_adjacent if adjacent else O.rope_rotate_half
    rng = np.random.default_rng(700 + b + t)
    qkv = make_bf16_activations(b * t, (h + 2 * kv) * d, 701 + t)
    pos = np.sort(rng.choice(s_max, t, replace=False)).astype(np.int64)
    ang = (pos[:, None] * (1.0 / 500000.0 ** (np.arange(0, d, 2) / d))[None, :]).astype(np.float32)
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    sentinel = 0x7FC1
    ck = np.full((b, kv, s_max, d), sentinel, np.uint16)
    cv = np.full((b, kv, s_max, d), sentinel, np.uint16)
    qd, ckd, cvd = torch.zeros((b, h, t, d), dtype=torch.int16, device="cuda"), _dev(ck), _dev(cv)
    xd, cd, sd, pd = _dev(qkv), _dev(cos), _dev(sin), _dev(pos)      # named: they must outlive the launch
    print(f"[case] rope_kv_store b={b} t={t} h={h} kv={kv} d={d} adjacent={adjacent}", flush=True)
    lib.ternaspmm_rope_kv_store(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 0, _vp(qd), _vp(ckd), _vp(cvd), b, t, h, kv, d,
                                s_max, adjacent, None)
    torch.cuda.synchronize()
    x = qkv.reshape(b, t, h + 2 * kv, d)
    want_q = rope(x[:, :, :h], cos[None, :, None], sin[None, :, None]).transpose(0, 2, 1, 3)
    want_k = rope(x[:, :, h:h + kv], cos[None, :, None], sin[None, :, None]).transpose(0, 2, 1, 3)
    want_v = x[:, :, h + kv:].transpose(0, 2, 1, 3)
    got_q = qd.cpu().numpy().view(np.uint16)
    got_k, got_v = ckd.cpu().numpy().view(np.uint16), cvd.cpu().numpy().view(np.uint16)
    assert (got_q == want_q).all()
    assert (got_k[:, :, pos] == want_k).all()
    assert (got_v[:, :, pos] == want_v).all()
    untouched = np.setdiff1d(np.arange(s_max), pos)
    assert (got_k[:, :, untouched] == sentinel).all() and (got_v[:, :, untouched] == sentinel).all()


@pytest.mark.parametrize("b,h,kv,d,s_max,n", [(1, 20, 5, 128, 256, 1), (1, 20, 5, 128, 256, 160), (8, 20, 5, 128, 512, 512),
                                              (2, 4, 2, 64, 40, 17), (1, 20, 5, 128, 4096, 4000),
                                              (2, 4, 2, 64, 1040, 1030), (8, 20, 5, 128, 1024, 1000), (1, 20, 5, 128, 1024, 3)])
@pytest.mark.parametrize("split", [False, True])
def test_decode_attention(lib, b, h, kv, d, s_max, n, split):
    """split: with a workspace and a cache of 1024 slots or more, the prefix of a head is spread over several
    workgroups and merged by the last one to arrive; two launches in a row on one workspace (the counters must
    be back at zero)."""
    q = make_bf16_activations(b * h, d, 710 + n).reshape(b, h, d)
    k = make_bf16_activations(b * kv * s_max, d, 711 + n).reshape(b, kv, s_max, d)
    v = make_bf16_activations(b * kv * s_max, d, 712 + n, outlier_frac=0.01).reshape(b, kv, s_max, d)
    pos = np.array([n - 1], np.int64)
    od = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    qd, kd, vd, pd = _dev(q), _dev(k), _dev(v), _dev(pos)            # named: they must outlive the launch
    ws = _attn_workspace(lib, b, h, d) if split else None
    print(f"[case] decode attention b={b} h={h} kv={kv} d={d} S={s_max} n={n} split={split}", flush=True)
    lib.ternaspmm_decode_attention(_vp(qd), _vp(kd), _vp(vd), _vp(pd), 0, _vp(od), b, h, kv, d, s_max, float(d) ** -0.5, _vp(ws), None)
    torch.cuda.synchronize()
    got = O.bf16_bits_to_f32(od.cpu().numpy().view(np.uint16)).reshape(b, h, d).astype(np.float64)
    want = O.attention_one_token(q, k, v, n, float(d) ** -0.5)
    # fp32 softmax and accumulation, bf16 output: relative to the largest output of the head
    tol = 2.0 ** -7 * np.abs(want).max(axis=-1, keepdims=True) + 1e-6
    assert (np.abs(got - want) <= tol).all(), float((np.abs(got - want) / tol).max())
    if split:
        counters = ws[:b * h * 4].view(torch.int32)
        assert int(counters.abs().sum().item()) == 0
        od2 = torch.zeros_like(od)
        lib.ternaspmm_decode_attention(_vp(qd), _vp(kd), _vp(vd), _vp(pd), 0, _vp(od2), b, h, kv, d, s_max, float(d) ** -0.5, _vp(ws), None)
        torch.cuda.synchronize()
        assert torch.equal(od, od2)                      # merged in split order: the same bits whoever arrives last


PREFILL_ATTENTION_CASES = [(1, 20, 5, 128, 160, 0, 128), (8, 20, 5, 128, 130, 0, 128), (2, 4, 2, 64, 64, 0, 23),
                           (2, 4, 2, 64, 300, 100, 50), (1, 20, 5, 128, 512, 300, 17), (3, 8, 8, 128, 40, 0, 1),
                           (1, 16, 2, 128, 200, 90, 70), (2, 8, 2, 64, 150, 0, 150), (1, 16, 2, 64, 96, 3, 40), (2, 3, 3, 64, 70, 0, 33),
                           (1, 6, 2, 128, 100, 0, 37), (1, 20, 5, 128, 1100, 0, 1090)]


def prefill_attention_case(lib, b, h, kv, d, s_max, first, t, check=True):
    """Runs one case of ternaspmm_prefill_attention, checks it against the oracle and returns the output bits."""
    q = make_bf16_activations(b * h * t, d, 720 + t).reshape(b, h, t, d)
    k = make_bf16_activations(b * kv * s_max, d, 721 + t).reshape(b, kv, s_max, d)
    v = make_bf16_activations(b * kv * s_max, d, 722 + t, outlier_frac=0.01).reshape(b, kv, s_max, d)
    k[:, :, first + t:] = 0x7FC0
    v[:, :, first + t:] = 0x7FC0
    pos = np.arange(first, first + t, dtype=np.int64)
    od = torch.full((b * t, h * d), 0x7FC0, dtype=torch.int16, device="cuda")
    qd, kd, vd, pd = _dev(q), _dev(k), _dev(v), _dev(pos)
    print(f"[case] prefill attention b={b} h={h} kv={kv} d={d} S={s_max} first={first} t={t}", flush=True)
    lib.ternaspmm_prefill_attention(_vp(qd), _vp(kd), _vp(vd), _vp(pd), 0, _vp(od), b, t, h, kv, d, s_max, float(d) ** -0.5, None)
    torch.cuda.synchronize()
    bits = od.cpu().numpy().view(np.uint16)
    if check:
        got = O.bf16_bits_to_f32(bits).reshape(b, t, h, d).astype(np.float64)
        want = O.attention_new_tokens(q, k, v, pos, float(d) ** -0.5)
        tol = 2.0 ** -7 * np.abs(want).max(axis=-1, keepdims=True) + 1e-6
        assert np.isfinite(got).all()
        assert (np.abs(got - want) <= tol).all(), float((np.abs(got - want) / tol).max())
    return bits


@pytest.mark.parametrize("b,h,kv,d,s_max,first,t", PREFILL_ATTENTION_CASES)
def test_prefill_attention(lib, b, h, kv, d, s_max, first, t):
    """T new tokens per sequence at the slots first .. first + T - 1, each attending over the cache up to its own
    slot (the prompt pass; with first > 0 a chunk appended to an existing prefix): against attention_one_token row by
    row, to the tolerance of the single-token kernel.  Slots past the newest token hold NaN bit patterns: nothing
    beyond a token's own slot may reach its output.  The cases cover 1, 2, 4 and 8 query heads per kv head (one
    workgroup per kv head), 3 (one wave per head), both head sizes, ragged last query blocks and a prefix of more than
    a thousand slots."""
    prefill_attention_case(lib, b, h, kv, d, s_max, first, t)


def _random_prefill_attention_shapes(count, seed):
    rng = np.random.default_rng(seed)
    shapes = []
    for _ in range(count):
        kv, group = int(rng.choice([1, 2, 3, 5])), int(rng.choice([1, 2, 3, 4, 8]))
        t = int(rng.choice([rng.integers(1, 17), rng.integers(17, 130), rng.integers(130, 400)]))
        first = int(rng.choice([0, rng.integers(1, 300)]))
        shapes.append((int(rng.integers(1, 4)), kv * group, kv, int(rng.choice([64, 128])), first + t + int(rng.integers(0, 40)), first, t))
    return shapes


@pytest.mark.parametrize("b,h,kv,d,s_max,first,t", _random_prefill_attention_shapes(12, 20260904))
def test_prefill_attention_random_shapes(lib, b, h, kv, d, s_max, first, t):
    """Seeded shapes nobody tuned for: 1 - 8 query heads per kv head (3: the one-wave-per-head kernel), 1 - 400 new tokens
    behind prefixes of 0 - 300 slots, caches that end anywhere."""
    prefill_attention_case(lib, b, h, kv, d, s_max, first, t)


def test_prefill_attention_kernels_give_the_same_bits(lib):
    """The grouped kernel (query heads of a kv head in one workgroup, keys / values through LDS) against the one-wave
    kernel, which a child process selects through the tuning override: same arithmetic in the same order, so the
    outputs must agree bit for bit."""
    import hashlib
    import os
    import subprocess
    import sys
    cases = [c for c in PREFILL_ATTENTION_CASES if c[1] // c[2] in (1, 2, 4, 8)][:8]
    mine = [hashlib.sha1(prefill_attention_case(lib, *c, check=False).tobytes()).hexdigest() for c in cases]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = ("import hashlib\nfrom ternainfer_amd import _lib\nfrom tests import test_gpu_prologue as P\nlib = _lib.load()\n"
            f"for c in {cases!r}:\n    print('bits', hashlib.sha1(P.prefill_attention_case(lib, *c, check=False).tobytes()).hexdigest(), flush=True)\n")
    r = subprocess.run([sys.executable, "-u", "-c", code], cwd=root, capture_output=True, text=True, timeout=300,
                       env={**os.environ, "TERNASPMM_TUNING": "1", "TERNASPMM_PREFILL_ATTN_GROUP": "0"})
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    theirs = [line.split()[1] for line in r.stdout.splitlines() if line.startswith("bits ")]
    assert theirs == mine, (theirs, mine)


def _attn_workspace(lib, b, h, d):
    nbytes = lib.ternaspmm_attention_workspace_bytes(b, h, d)
    assert nbytes > 0
    return torch.zeros(nbytes, dtype=torch.int8, device="cuda")


# ------------------------------------------------------------------ prologue inside the small-M linear
def _bf16_key(b):
    b = b.astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)


@pytest.mark.parametrize("m", [1, 2, 3, 4, 8, 11, 16])
@pytest.mark.parametrize("n,k,ws_num,res", [(3840, 2560, 3, True), (2560, 2560, 1, False), (13824, 2560, 2, True),
                                            (256, 192, 1, True), (320, 64, 2, False), (4160, 128, 1, False)])
def test_fused_prologue_linear(lib, m, n, k, ws_num, res):
    _check_fused_prologue_linear(lib, m, n, k, ws_num, res)


@pytest.mark.parametrize("m", [1, 3, 8])
@pytest.mark.parametrize("n,k,ws_num", [(2560, 6912, 1), (320, 8192, 2), (4096, 3136, 1)])
def test_fused_prologue_linear_long_rows(lib, m, n, k, ws_num):
    """Without a residual, up to 8 rows and 4096 outputs the entry point takes rows of up to 8192 columns."""
    _check_fused_prologue_linear(lib, m, n, k, ws_num, False)


def _check_fused_prologue_linear(lib, m, n, k, ws_num, res):
    """One launch: residual add -> norm -> quantise -> ternary matmul -> epilogue.  The published h is exact,
    s and q are what the oracle quantiser gives for a norm output within one bf16 step of the float64 one,
    and the matmul + epilogue on the kernel's own (q, s) is bit-exact."""
    from tests._util import DeviceFormat, make_ternary
    w = make_ternary(n, k, 0.40, 800 + m + n)
    fmt = DeviceFormat(w)
    packed = torch.empty(n * k // 16, dtype=torch.int32, device="cuda")
    lib.ternaspmm_repack(_vp(fmt.bm), _vp(fmt.off), _vp(fmt.med), _vp(fmt.vals), _vp(packed), n, k, None)
    x = make_bf16_activations(m, k, 801 + m + k, outlier_frac=0.01)
    r = make_bf16_activations(m, k, 802 + m + k) if res else None
    g = _weight(k, 803 + k)
    ws = O.f32_to_bf16_bits(np.array([1.25, 0.75, 1.5, 0.0], np.float32))
    xd, gd, wsd = _dev(x), _dev(g), _dev(ws)
    rd = _dev(r) if res else None
    hd = torch.zeros((m, k), dtype=torch.int16, device="cuda") if res else None
    od = torch.zeros((m, n), dtype=torch.int16, device="cuda")
    qd = torch.zeros((m, k), dtype=torch.int8, device="cuda")
    sd = torch.zeros(m, dtype=torch.int16, device="cuda")
    print(f"[case] fused prologue linear m={m} n={n} k={k} ws_num={ws_num} res={res}", flush=True)
    done = lib.bitlinear_TernaSpMM_packed_fused(_vp(xd), _vp(rd), _vp(hd), _vp(gd), 1e-5, _vp(packed), _vp(od), _vp(wsd), ws_num,
                                                _vp(qd), _vp(sd), m, n, k, None)
    torch.cuda.synchronize()
    assert done == 1
    h = x
    if res:
        h = O.residual_add(x, r)
        assert (hd.cpu().numpy().view(np.uint16) == h).all()
    q, s = qd.cpu().numpy(), sd.cpu().numpy().view(np.uint16)
    y64 = O.rmsnorm(h, g, 1e-5)
    _, s_want = O.quant_input(y64)
    assert np.abs(_bf16_key(s) - _bf16_key(s_want)).max() <= 1
    q_ref = np.clip(np.rint(O.bf16_bits_to_f32(y64) * O.bf16_bits_to_f32(s)[:, None]), -128, 127)
    dq = np.abs(q.astype(np.int32) - q_ref.astype(np.int32))
    assert dq.max() <= 1 and (dq != 0).mean() < 0.02
    want = O.spmm_i8(q, w, s, ws, ws_num, 0)
    assert (od.cpu().numpy().view(np.uint16) == want).all()
    # optional outputs off: same result
    od2 = torch.zeros_like(od)
    hd2 = torch.zeros_like(hd) if res else None
    assert lib.bitlinear_TernaSpMM_packed_fused(_vp(xd), _vp(rd), _vp(hd2), _vp(gd), 1e-5, _vp(packed), _vp(od2), _vp(wsd),
                                                ws_num, None, None, m, n, k, None) == 1
    torch.cuda.synchronize()
    assert torch.equal(od, od2)


@pytest.mark.parametrize("mode", [O.QUANT_COMPILED, O.QUANT_EAGER])
def test_quant_modes_of_the_prologue_kernels(lib, mode):
    """ternaspmm_quant_mode: the reference's other evaluations of quant_input (model.py:120-123; the @torch.compile'd
    method as shipped, and eager mode on bf16 tensors).  The norm kernels' (q, s) must be the oracle's for that mode
    on the kernel's own norm output, bit for bit; the fused linear's must be that mode's for a norm output within one
    bf16 step, with the matmul on them bit-exact; and the mode must really change the integers."""
    from tests._util import DeviceFormat, make_ternary
    assert lib.ternaspmm_quant_mode(-1) == O.QUANT_ROUNDED
    x = make_bf16_activations(37, 2560, 640, outlier_frac=0.01)
    x13 = make_bf16_activations(9, 2 * 6912, 641, outlier_frac=0.01)
    w, wf = _weight(2560, 642), _weight(6912, 643)
    _, _, q0, _ = _run(lib, x, w, 1e-5)
    n, k, m = 2560, 2560, 8
    wt = make_ternary(n, k, 0.40, 644)
    fmt = DeviceFormat(wt)
    packed = torch.empty(n * k // 16, dtype=torch.int32, device="cuda")
    lib.ternaspmm_repack(_vp(fmt.bm), _vp(fmt.off), _vp(fmt.med), _vp(fmt.vals), _vp(packed), n, k, None)
    ws = O.f32_to_bf16_bits(np.array([1.25, 0.0, 0.0, 0.0], np.float32))
    assert lib.ternaspmm_quant_mode(mode) == O.QUANT_ROUNDED
    try:
        print(f"[case] quant mode {mode}: norm kernels", flush=True)
        _, y, q, s = _run(lib, x, w, 1e-5)
        want_q, want_s = O.quant_input(y, mode)
        assert (s == want_s).all() and (q == want_q).all()
        assert 0 < (q != q0).mean() < 0.2                           # not the default rule's integers
        _, y, q, s = _run(lib, x13, wf, 1e-5, glu=True)
        want_q, want_s = O.quant_input(y, mode)
        assert (s == want_s).all() and (q == want_q).all()
        for mm in (1, m):
            print(f"[case] quant mode {mode}: fused prologue linear m={mm}", flush=True)
            xs = x[:mm]
            xd, gd, wsd = _dev(xs), _dev(w), _dev(ws)
            od = torch.zeros((mm, n), dtype=torch.int16, device="cuda")
            qd = torch.zeros((mm, k), dtype=torch.int8, device="cuda")
            sd = torch.zeros(mm, dtype=torch.int16, device="cuda")
            assert lib.bitlinear_TernaSpMM_packed_fused(_vp(xd), None, None, _vp(gd), 1e-5, _vp(packed), _vp(od), _vp(wsd), 1,
                                                        _vp(qd), _vp(sd), mm, n, k, None) == 1
            torch.cuda.synchronize()
            qk, sk = qd.cpu().numpy(), sd.cpu().numpy().view(np.uint16)
            q_ref, s_ref = O.quant_input(O.rmsnorm(xs, w, 1e-5), mode)
            assert np.abs(_bf16_key(sk) - _bf16_key(s_ref)).max() <= 1
            same_s = sk == s_ref                                     # rows whose scale agrees: the integers may differ only where y does
            dq = np.abs(qk.astype(np.int32) - q_ref.astype(np.int32))[same_s]
            assert dq.size and dq.max() <= 1 and (dq != 0).mean() < 0.02
            assert (od.cpu().numpy().view(np.uint16) == O.spmm_i8(qk, wt, sk, ws, 1, 0)).all()
    finally:
        lib.ternaspmm_quant_mode(O.QUANT_ROUNDED)
    _, _, q1, _ = _run(lib, x, w, 1e-5)
    assert (q1 == q0).all()


def test_fused_prologue_linear_declines_what_it_cannot_do(lib):
    z = torch.zeros(64, dtype=torch.int32, device="cuda")
    # declined before any argument is read: the buffers here are far smaller than the shapes
    for m, n, k in [(17, 256, 192), (8, 2560, 13824), (16, 2560, 6912), (8, 13824, 3136)]:
        assert lib.bitlinear_TernaSpMM_packed_fused(_vp(z), None, None, _vp(z), 1e-5, _vp(z), _vp(z), _vp(z), 1, None, None,
                                                    m, n, k, None) == 0


def test_rmsnorm_linear_wrapper_matches_two_launch_sequence(lib):
    """Wrapper: fused where supported, two launches elsewhere; both agree with the two-launch sequence up to
    the rare int8 flips a one-step difference in the norm output causes."""
    import ternainfer_amd as T
    from tests._util import make_ternary
    for n, k, m in [(256, 320, 1), (256, 6912, 1), (256, 320, 8)]:
        w = make_ternary(n, k, 0.4, 850 + k + m)
        vals, off, med, bm = [t.cuda() for t in T.compress_weight(torch.from_numpy(w))]
        packed = T.repack_weight(vals, off, med, bm, n, k)
        xt = torch.from_numpy(make_bf16_activations(m, k, 851).view(np.int16)).cuda().view(torch.bfloat16)
        rt = torch.from_numpy(make_bf16_activations(m, k, 852).view(np.int16)).cuda().view(torch.bfloat16)
        gt = torch.from_numpy(_weight(k, 853).view(np.int16)).cuda().view(torch.bfloat16)
        ws = torch.tensor([1.25, 0, 0, 0], dtype=torch.bfloat16, device="cuda")
        out, h = T.rmsnorm_linear_packed(xt, gt, 1e-5, packed, ws, 1, n, residual=rt)
        xq, s, h2 = T.rmsnorm_quant(xt, gt, 1e-5, residual=rt)
        out2 = T.TernaInfer_linear_packed(xq, packed, s, ws, 1, n)
        assert torch.equal(h, h2)
        err = (out.float() - out2.float()).abs().max().item()
        assert err <= 2e-2 * out2.float().abs().max().item()


@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("n,f,ws_num", [(2560, 6912, 1), (256, 192, 2), (320, 7168, 1)])
def test_fused_gate_prologue_linear(lib, n, f, ws_num, m):
    """Up to four rows: squared_relu(x1) * x3 -> norm -> quantise -> matmul in one launch; same bars as above."""
    from tests._util import DeviceFormat, make_ternary
    w = make_ternary(n, f, 0.40, 870 + n)
    fmt = DeviceFormat(w)
    packed = torch.empty(n * f // 16, dtype=torch.int32, device="cuda")
    lib.ternaspmm_repack(_vp(fmt.bm), _vp(fmt.off), _vp(fmt.med), _vp(fmt.vals), _vp(packed), n, f, None)
    x13 = make_bf16_activations(m, 2 * f, 871 + f + m, outlier_frac=0.01)
    g = _weight(f, 872)
    ws = O.f32_to_bf16_bits(np.array([1.25, 0.75, 0.0, 0.0], np.float32))
    xd, gd, wsd = _dev(x13), _dev(g), _dev(ws)
    od = torch.zeros((m, n), dtype=torch.int16, device="cuda")
    qd = torch.zeros((m, f), dtype=torch.int8, device="cuda")
    sd = torch.zeros(m, dtype=torch.int16, device="cuda")
    print(f"[case] fused gate prologue linear m={m} n={n} f={f}", flush=True)
    assert lib.bitlinear_TernaSpMM_packed_fused_glu(_vp(xd), _vp(gd), 1e-5, _vp(packed), _vp(od), _vp(wsd), ws_num, _vp(qd),
                                                    _vp(sd), m, n, f, None) == 1
    torch.cuda.synchronize()
    q, s = qd.cpu().numpy(), sd.cpu().numpy().view(np.uint16)
    y64 = O.rmsnorm(O.relu2_mul(x13), g, 1e-5)
    _, s_want = O.quant_input(y64)
    assert np.abs(_bf16_key(s) - _bf16_key(s_want)).max() <= 1
    q_ref = np.clip(np.rint(O.bf16_bits_to_f32(y64) * O.bf16_bits_to_f32(s)[:, None]), -128, 127)
    dq = np.abs(q.astype(np.int32) - q_ref.astype(np.int32))
    assert dq.max() <= 1 and (dq != 0).mean() < 0.02
    assert (od.cpu().numpy().view(np.uint16) == O.spmm_i8(q, w, s, ws, ws_num, 0)).all()
    z = torch.zeros(64, dtype=torch.int32, device="cuda")
    assert lib.bitlinear_TernaSpMM_packed_fused_glu(_vp(z), _vp(z), 1e-5, _vp(z), _vp(z), _vp(z), 1, None, None, 5, n, f, None) == 0


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("adjacent", [0, 1])
@pytest.mark.parametrize("b,h,kv,d,s_max,n", [(1, 20, 5, 128, 256, 1), (1, 20, 5, 128, 256, 160), (8, 20, 5, 128, 300, 290),
                                              (2, 4, 2, 64, 40, 17), (1, 20, 5, 128, 600, 513), (1, 20, 5, 128, 2048, 1500),
                                              (2, 4, 2, 64, 1024, 1)])
def test_rope_decode_attention_equals_the_two_launches(lib, b, h, kv, d, s_max, n, adjacent, split):
    """One launch (RoPE + cache write + attention) against ternaspmm_rope_kv_store followed by
    ternaspmm_decode_attention on the same inputs: outputs and both caches bit-identical."""
    rng = np.random.default_rng(720 + n)
    qkv = make_bf16_activations(b, (h + 2 * kv) * d, 721 + n)
    k0 = make_bf16_activations(b * kv * s_max, d, 722 + n).reshape(b, kv, s_max, d)
    v0 = make_bf16_activations(b * kv * s_max, d, 723 + n, outlier_frac=0.01).reshape(b, kv, s_max, d)
    pos = np.array([n - 1], np.int64)
    ang = (pos[:, None] * (1.0 / 500000.0 ** (np.arange(0, d, 2) / d))[None, :]).astype(np.float32)
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    xd, cd, sd, pd = _dev(qkv), _dev(cos), _dev(sin), _dev(pos)
    scale = float(d) ** -0.5
    ws1 = _attn_workspace(lib, b, h, d) if split else None
    ws2 = _attn_workspace(lib, b, h, d) if split else None
    # two launches
    ck1, cv1 = _dev(k0), _dev(v0)
    q1 = torch.zeros((b, h, 1, d), dtype=torch.int16, device="cuda")
    o1 = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    lib.ternaspmm_rope_kv_store(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 0, _vp(q1), _vp(ck1), _vp(cv1), b, 1, h, kv, d, s_max, adjacent, None)
    lib.ternaspmm_decode_attention(_vp(q1), _vp(ck1), _vp(cv1), _vp(pd), 0, _vp(o1), b, h, kv, d, s_max, scale, _vp(ws1), None)
    # one launch
    ck2, cv2 = _dev(k0), _dev(v0)
    o2 = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    print(f"[case] rope + decode attention b={b} h={h} kv={kv} d={d} S={s_max} n={n} adjacent={adjacent}", flush=True)
    lib.ternaspmm_rope_decode_attention(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 0, _vp(ck2), _vp(cv2), _vp(o2), b, h, kv, d, s_max,
                                        scale, adjacent, _vp(ws2), None)
    torch.cuda.synchronize()
    assert torch.equal(ck1, ck2) and torch.equal(cv1, cv2)
    assert torch.equal(o1, o2)


@pytest.mark.parametrize("b,h,kv,d,s_max,n", [(1, 20, 5, 128, 384, 200), (8, 20, 5, 128, 384, 300), (2, 4, 2, 64, 40, 17)])
def test_rope_decode_attention_with_prefetch_regions(lib, b, h, kv, d, s_max, n):
    """The variant with prefetch workgroups: same output and caches as the plain entry point, bit for bit, and the
    prefetched regions (sizes that are and are not multiples of the unit, a unit larger than the region, a
    region the call must skip) are left untouched."""
    qkv = make_bf16_activations(b, (h + 2 * kv) * d, 931 + n)
    k0 = make_bf16_activations(b * kv * s_max, d, 932 + n).reshape(b, kv, s_max, d)
    v0 = make_bf16_activations(b * kv * s_max, d, 933 + n).reshape(b, kv, s_max, d)
    pos = np.array([n - 1], np.int64)
    ang = (pos[:, None] * (1.0 / 500000.0 ** (np.arange(0, d, 2) / d))[None, :]).astype(np.float32)
    xd, cd, sd, pd = _dev(qkv), _dev(np.cos(ang).astype(np.float32)), _dev(np.sin(ang).astype(np.float32)), _dev(pos)
    scale = float(d) ** -0.5
    ck1, cv1, ck2, cv2 = _dev(k0), _dev(v0), _dev(k0), _dev(v0)
    o1 = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    o2 = torch.zeros_like(o1)
    gen = torch.Generator(device="cuda").manual_seed(5)
    regions = [torch.randint(-2 ** 31, 2 ** 31 - 1, (nwords,), dtype=torch.int32, device="cuda", generator=gen)
               for nwords in (40 * 2560, 3 * 2560 + 36, 64, 4096)]
    before = [r.clone() for r in regions]
    units = [10240, 10240, 40960, 27648]
    count = len(regions) + 1
    ptrs = (ctypes.c_void_p * count)(*([r.data_ptr() for r in regions] + [None]))           # the last one is skipped
    sizes = (ctypes.c_longlong * count)(*([r.numel() * 4 for r in regions] + [1024]))
    unit_arr = (ctypes.c_longlong * count)(*(units + [16]))
    lib.ternaspmm_rope_decode_attention(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 0, _vp(ck1), _vp(cv1), _vp(o1), b, h, kv, d, s_max,
                                        scale, 1, None, None)
    print(f"[case] rope + decode attention with prefetch b={b} h={h} d={d} n={n}", flush=True)
    lib.ternaspmm_rope_decode_attention_prefetch(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 0, _vp(ck2), _vp(cv2), _vp(o2), b, h, kv, d,
                                                 s_max, scale, 1, None, ptrs, sizes, unit_arr, count, None)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2) and torch.equal(ck1, ck2) and torch.equal(cv1, cv2)
    assert all(torch.equal(r, r0) for r, r0 in zip(regions, before))


@pytest.mark.parametrize("b,v,hist", [(1, 128256, 4), (8, 128256, 3), (3, 1003, 2), (37, 4096, 5), (2, 64, 1), (300, 520, 2)])
def test_greedy_step(lib, b, v, hist):
    """argmax + history append + counters in one launch, several launches in a row on one state: the
    same tokens as the one-row-per-workgroup argmax (ties, -inf, NaN, unaligned rows), the history
    filled up to its length and not beyond, counters advanced every time."""
    import ternainfer_amd as T
    rng = np.random.default_rng(7000 + b + v)
    state = T.greedy_step_state(b)
    tok = torch.full((b, 1), -1, dtype=torch.int64, device="cuda")
    history = torch.full((b, hist + 1), -7, dtype=torch.int64, device="cuda")[:, :hist].contiguous()
    counters = torch.tensor([40, 0], dtype=torch.int64, device="cuda")
    want_hist = np.full((b, hist), -7, np.int64)
    for launch in range(hist + 2):
        xf = O.bf16_bits_to_f32(O.f32_to_bf16_bits(rng.standard_normal((b, v)).astype(np.float32)))
        if v >= 64:
            xf[0, 17] = xf[0, v - 3] = 9.0                                       # a tie across chunks: the lower index wins
            xf[-1, 3] = -np.inf
            xf[-1, 11] = np.nan
        if launch == 1:
            xf[0, :] = -np.inf                                                   # nothing ever wins: index 0
        x = O.f32_to_bf16_bits(xf)
        xf = O.bf16_bits_to_f32(x)
        want = np.array([0 if np.all(np.isneginf(r[~np.isnan(r)])) else int(np.flatnonzero(r == np.nanmax(r))[0]) for r in xf], np.int64)
        xd = _dev(x).view(torch.bfloat16)
        print(f"[case] greedy_step b={b} v={v} launch={launch}", flush=True)
        T.greedy_step(xd, tok, history, counters, state)
        torch.cuda.synchronize()
        assert (tok.cpu().numpy().ravel() == want).all()
        assert (T.argmax_rows(xd).cpu().numpy().ravel() == want).all()
        if launch < hist:
            want_hist[:, launch] = want
        assert (history.cpu().numpy() == want_hist).all()
        assert counters.cpu().tolist() == [41 + launch, 1 + launch]
        assert int(state[0].item()) == 0
    # without history and counters: only the tokens
    T.greedy_step(xd, tok.fill_(-1), None, None, state)
    torch.cuda.synchronize()
    assert (tok.cpu().numpy().ravel() == want).all()


# ------------------------------------------------------------------ per-sequence positions (per_sequence = 1)
def _angles(pos, d):
    ang = (pos.reshape(-1)[:, None] * (1.0 / 500000.0 ** (np.arange(0, d, 2) / d))[None, :]).astype(np.float32)
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


@pytest.mark.parametrize("adjacent", [0, 1])
@pytest.mark.parametrize("b,t,h,kv,d,s_max", [(3, 1, 20, 5, 128, 64), (2, 7, 4, 2, 64, 40), (4, 3, 4, 2, 24, 16)])
def test_rope_kv_store_per_sequence(lib, b, t, h, kv, d, s_max, adjacent):
    """Every sequence at its own cache slots and angles (pos [B][T], cos / sin [B][T][D/2]): sequence by sequence
    against the rotation of the oracle, rows of other slots untouched."""
    rope = O.rope_adjacent if adjacent else O.rope_rotate_half
    rng = np.random.default_rng(1700 + b + t)
    qkv = make_bf16_activations(b * t, (h + 2 * kv) * d, 1701 + t)
    pos = np.stack([np.sort(rng.choice(s_max, t, replace=False)) for _ in range(b)]).astype(np.int64)      # [B][T]
    cos, sin = _angles(pos, d)                                                                               # [B*T][D/2]
    sentinel = 0x7FC1
    ck = np.full((b, kv, s_max, d), sentinel, np.uint16)
    cv = np.full((b, kv, s_max, d), sentinel, np.uint16)
    qd, ckd, cvd = torch.zeros((b, h, t, d), dtype=torch.int16, device="cuda"), _dev(ck), _dev(cv)
    xd, cd, sd, pd = _dev(qkv), _dev(cos), _dev(sin), _dev(pos)
    print(f"[case] rope_kv_store per sequence b={b} t={t} h={h} kv={kv} d={d} adjacent={adjacent}", flush=True)
    lib.ternaspmm_rope_kv_store(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(qd), _vp(ckd), _vp(cvd), b, t, h, kv, d,
                                s_max, adjacent, None)
    torch.cuda.synchronize()
    x = qkv.reshape(b, t, h + 2 * kv, d)
    c4, s4 = cos.reshape(b, t, 1, d // 2), sin.reshape(b, t, 1, d // 2)
    want_q = rope(x[:, :, :h], c4, s4).transpose(0, 2, 1, 3)
    want_k = rope(x[:, :, h:h + kv], c4, s4).transpose(0, 2, 1, 3)
    want_v = x[:, :, h + kv:].transpose(0, 2, 1, 3)
    got_q = qd.cpu().numpy().view(np.uint16)
    got_k, got_v = ckd.cpu().numpy().view(np.uint16), cvd.cpu().numpy().view(np.uint16)
    assert (got_q == want_q).all()
    for i in range(b):
        assert (got_k[i][:, pos[i]] == want_k[i]).all() and (got_v[i][:, pos[i]] == want_v[i]).all()
        untouched = np.setdiff1d(np.arange(s_max), pos[i])
        assert (got_k[i][:, untouched] == sentinel).all() and (got_v[i][:, untouched] == sentinel).all()


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("b,h,kv,d,s_max,lens", [(3, 20, 5, 128, 256, (1, 160, 77)), (8, 20, 5, 128, 1024, (1000, 3, 512, 17, 1024, 64, 65, 700)),
                                                 (2, 4, 2, 64, 1040, (1030, 12))])
def test_decode_attention_per_sequence(lib, b, h, kv, d, s_max, lens, split):
    """Sequences of different prefix lengths in one call (pos [B]): every sequence against the oracle at its own
    length, and bit-identical to a call of its own with the shared-position form."""
    _decode_attention_per_sequence_case(lib, b, h, kv, d, s_max, lens, split)


def _random_attention_shapes(count, seed):
    """Seeded shapes nobody tuned for: 1 - 16 sequences, 1 - 8 query heads per kv head, caches of 1 - 1300 slots, prefix
    lengths anywhere in them (always one sequence at a single token and one at the full cache when there is room)."""
    rng = np.random.default_rng(seed)
    shapes = []
    for _ in range(count):
        b = int(rng.integers(1, 17))
        kv, group = int(rng.choice([1, 2, 5, 8])), int(rng.choice([1, 2, 4, 8]))
        d = int(rng.choice([64, 128]))
        s_max = int(rng.choice([rng.integers(1, 65), rng.integers(65, 400), rng.integers(400, 1301)]))
        lens = [int(x) for x in rng.integers(1, s_max + 1, b)]
        lens[0] = s_max
        if b > 1:
            lens[-1] = 1
        shapes.append((b, kv * group, kv, d, s_max, tuple(lens)))
    return shapes


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("b,h,kv,d,s_max,lens", _random_attention_shapes(12, 20260902))
def test_decode_attention_random_shapes(lib, b, h, kv, d, s_max, lens, split):
    _decode_attention_per_sequence_case(lib, b, h, kv, d, s_max, lens, split)


def _decode_attention_per_sequence_case(lib, b, h, kv, d, s_max, lens, split):
    q = make_bf16_activations(b * h, d, 1710 + b).reshape(b, h, d)
    k = make_bf16_activations(b * kv * s_max, d, 1711 + b).reshape(b, kv, s_max, d)
    v = make_bf16_activations(b * kv * s_max, d, 1712 + b, outlier_frac=0.01).reshape(b, kv, s_max, d)
    pos = np.array(lens, np.int64) - 1
    od = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    qd, kd, vd, pd = _dev(q), _dev(k), _dev(v), _dev(pos)
    ws = _attn_workspace(lib, b, h, d) if split else None
    print(f"[case] decode attention per sequence b={b} h={h} d={d} S={s_max} lens={lens} split={split}", flush=True)
    lib.ternaspmm_decode_attention(_vp(qd), _vp(kd), _vp(vd), _vp(pd), 1, _vp(od), b, h, kv, d, s_max, float(d) ** -0.5, _vp(ws), None)
    torch.cuda.synchronize()
    got = O.bf16_bits_to_f32(od.cpu().numpy().view(np.uint16)).reshape(b, h, d).astype(np.float64)
    for i in range(b):
        want = O.attention_one_token(q[i:i + 1], k[i:i + 1], v[i:i + 1], lens[i], float(d) ** -0.5)[0]
        tol = 2.0 ** -7 * np.abs(want).max(axis=-1, keepdims=True) + 1e-6
        assert (np.abs(got[i] - want) <= tol).all(), (i, float((np.abs(got[i] - want) / tol).max()))
    # the same sequences one at a time, shared-position form: the same bits (a head's work does not depend on the batch)
    ws1 = _attn_workspace(lib, 1, h, d) if split else None
    for i in range(b):
        o1 = torch.zeros((1, h * d), dtype=torch.int16, device="cuda")
        p1 = _dev(pos[i:i + 1])
        lib.ternaspmm_decode_attention(_vp(qd[i:i + 1]), _vp(kd[i:i + 1]), _vp(vd[i:i + 1]), _vp(p1), 0, _vp(o1), 1, h, kv, d, s_max,
                                       float(d) ** -0.5, _vp(ws1), None)
        torch.cuda.synchronize()
        # (with a workspace the split count depends on B, and above 512 heads per call the workgroups are four waves wide
        # instead of eight: other summation orders, checked against the oracle above only)
        if not split and b * h <= 512:
            assert torch.equal(o1[0], od[i])
    if split:
        assert int(ws[:b * h * 4].view(torch.int32).abs().sum().item()) == 0


@pytest.mark.parametrize("b,h,kv,d,s_max,firsts,t", [(3, 20, 5, 128, 200, (0, 60, 17), 40), (2, 4, 2, 64, 300, (100, 0), 50),
                                                    (4, 8, 8, 128, 64, (5, 0, 33, 20), 1)])
def test_prefill_attention_per_sequence(lib, b, h, kv, d, s_max, firsts, t):
    """T new tokens per sequence, sequence b at the slots firsts[b] .. firsts[b] + T - 1 (pos [B][T]); slots past each
    sequence's newest token hold NaN bit patterns."""
    q = make_bf16_activations(b * h * t, d, 1720 + t).reshape(b, h, t, d)
    k = make_bf16_activations(b * kv * s_max, d, 1721 + t).reshape(b, kv, s_max, d)
    v = make_bf16_activations(b * kv * s_max, d, 1722 + t, outlier_frac=0.01).reshape(b, kv, s_max, d)
    for i in range(b):
        k[i, :, firsts[i] + t:] = 0x7FC0
        v[i, :, firsts[i] + t:] = 0x7FC0
    pos = np.stack([np.arange(f, f + t) for f in firsts]).astype(np.int64)
    od = torch.full((b * t, h * d), 0x7FC0, dtype=torch.int16, device="cuda")
    qd, kd, vd, pd = _dev(q), _dev(k), _dev(v), _dev(pos)
    print(f"[case] prefill attention per sequence b={b} h={h} d={d} S={s_max} firsts={firsts} t={t}", flush=True)
    lib.ternaspmm_prefill_attention(_vp(qd), _vp(kd), _vp(vd), _vp(pd), 1, _vp(od), b, t, h, kv, d, s_max, float(d) ** -0.5, None)
    torch.cuda.synchronize()
    got = O.bf16_bits_to_f32(od.cpu().numpy().view(np.uint16)).reshape(b, t, h, d).astype(np.float64)
    assert np.isfinite(got).all()
    for i in range(b):
        want = O.attention_new_tokens(q[i:i + 1], k[i:i + 1], v[i:i + 1], pos[i], float(d) ** -0.5)[0]
        tol = 2.0 ** -7 * np.abs(want).max(axis=-1, keepdims=True) + 1e-6
        assert (np.abs(got[i] - want) <= tol).all(), (i, float((np.abs(got[i] - want) / tol).max()))


@pytest.mark.parametrize("prefetch", [False, True])
@pytest.mark.parametrize("adjacent", [0, 1])
@pytest.mark.parametrize("b,h,kv,d,s_max,lens", [(3, 20, 5, 128, 300, (290, 1, 45)), (2, 4, 2, 64, 40, (17, 40)),
                                                 (8, 20, 5, 128, 384, (200, 201, 1, 384, 100, 7, 300, 64))])
def test_rope_decode_attention_per_sequence(lib, b, h, kv, d, s_max, lens, adjacent, prefetch):
    """One launch with per-sequence positions against ternaspmm_rope_kv_store + ternaspmm_decode_attention with the
    same positions (outputs and both caches bit-identical), and against one shared-position call per sequence."""
    qkv = make_bf16_activations(b, (h + 2 * kv) * d, 1731 + b)
    k0 = make_bf16_activations(b * kv * s_max, d, 1732 + b).reshape(b, kv, s_max, d)
    v0 = make_bf16_activations(b * kv * s_max, d, 1733 + b, outlier_frac=0.01).reshape(b, kv, s_max, d)
    pos = np.array(lens, np.int64) - 1
    cos, sin = _angles(pos, d)                                                    # [B][D/2]
    xd, cd, sd, pd = _dev(qkv), _dev(cos), _dev(sin), _dev(pos)
    scale = float(d) ** -0.5
    ck1, cv1, ck2, cv2 = _dev(k0), _dev(v0), _dev(k0), _dev(v0)
    q1 = torch.zeros((b, h, 1, d), dtype=torch.int16, device="cuda")
    o1 = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    o2 = torch.zeros_like(o1)
    lib.ternaspmm_rope_kv_store(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(q1), _vp(ck1), _vp(cv1), b, 1, h, kv, d, s_max, adjacent, None)
    lib.ternaspmm_decode_attention(_vp(q1), _vp(ck1), _vp(cv1), _vp(pd), 1, _vp(o1), b, h, kv, d, s_max, scale, None, None)
    print(f"[case] rope + decode attention per sequence b={b} h={h} d={d} lens={lens} adjacent={adjacent} prefetch={prefetch}", flush=True)
    if prefetch:
        region = torch.zeros(40 * 2560, dtype=torch.int32, device="cuda")
        ptrs = (ctypes.c_void_p * 1)(region.data_ptr())
        sizes = (ctypes.c_longlong * 1)(region.numel() * 4)
        units = (ctypes.c_longlong * 1)(10240)
        lib.ternaspmm_rope_decode_attention_prefetch(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(ck2), _vp(cv2), _vp(o2), b, h, kv, d,
                                                     s_max, scale, adjacent, None, ptrs, sizes, units, 1, None)
    else:
        lib.ternaspmm_rope_decode_attention(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(ck2), _vp(cv2), _vp(o2), b, h, kv, d, s_max,
                                            scale, adjacent, None, None)
    torch.cuda.synchronize()
    assert torch.equal(ck1, ck2) and torch.equal(cv1, cv2) and torch.equal(o1, o2)
    for i in range(b):                                   # sequence i alone, shared-position form
        ck3, cv3 = _dev(k0[i:i + 1]), _dev(v0[i:i + 1])
        o3 = torch.zeros((1, h * d), dtype=torch.int16, device="cuda")
        c3, s3, p3 = _dev(cos[i:i + 1]), _dev(sin[i:i + 1]), _dev(pos[i:i + 1])
        lib.ternaspmm_rope_decode_attention(_vp(xd[i:i + 1]), _vp(c3), _vp(s3), _vp(p3), 0, _vp(ck3), _vp(cv3), _vp(o3), 1, h, kv, d,
                                            s_max, scale, adjacent, None, None)
        torch.cuda.synchronize()
        assert torch.equal(o3[0], o2[i]) and torch.equal(ck3[0], ck2[i]) and torch.equal(cv3[0], cv2[i])


# ------------------------------------------------------------------ split attention with the merge left to the next launch
def _partial_buffer(lib, b, h, d):
    nbytes = lib.ternaspmm_attention_partial_bytes(b, h, d)
    assert nbytes > 0
    return torch.full((nbytes // 4,), float("nan"), dtype=torch.float32, device="cuda")       # needs no initialisation


@pytest.mark.parametrize("per_seq", [0, 1])
@pytest.mark.parametrize("splits", [1, 2, 4, 8])
@pytest.mark.parametrize("b,h,kv,d,s_max,n", [(1, 20, 5, 128, 384, 200), (1, 20, 5, 128, 4096, 4000), (2, 4, 2, 64, 300, 17),
                                              (3, 8, 8, 128, 64, 1), (1, 20, 5, 128, 2048, 1029)])
def test_rope_decode_attention_partial_and_merge(lib, b, h, kv, d, s_max, n, splits, per_seq):
    """The split attention that leaves the merge to the next launch + the merge kernel: caches bit-identical to
    ternaspmm_rope_decode_attention, output within the attention tolerance of the oracle (splits change the order
    of the sums); a prefix shorter than the splits leaves empty splits, which the merge must weigh with zero; and
    with a prefetch region the launch gives the same bits."""
    lens = [max(1, n - 7 * i) for i in range(b)] if per_seq else [n] * b
    qkv = make_bf16_activations(b, (h + 2 * kv) * d, 1801 + n)
    k0 = make_bf16_activations(b * kv * s_max, d, 1802 + n).reshape(b, kv, s_max, d)
    v0 = make_bf16_activations(b * kv * s_max, d, 1803 + n, outlier_frac=0.01).reshape(b, kv, s_max, d)
    pos = (np.array(lens, np.int64) - 1) if per_seq else np.array([n - 1], np.int64)
    cos, sin = _angles(pos, d)
    xd, cd, sd, pd = _dev(qkv), _dev(cos), _dev(sin), _dev(pos)
    scale = float(d) ** -0.5
    ck1, cv1, ck2, cv2, ck3, cv3 = _dev(k0), _dev(v0), _dev(k0), _dev(v0), _dev(k0), _dev(v0)
    o1 = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    o2, o3 = torch.zeros_like(o1), torch.zeros_like(o1)
    lib.ternaspmm_rope_decode_attention(_vp(xd), _vp(cd), _vp(sd), _vp(pd), per_seq, _vp(ck1), _vp(cv1), _vp(o1), b, h, kv, d, s_max,
                                        scale, 1, None, None)
    part = _partial_buffer(lib, b, h, d)
    print(f"[case] attention partial + merge b={b} h={h} d={d} S={s_max} n={n} splits={splits} per_seq={per_seq}", flush=True)
    lib.ternaspmm_rope_decode_attention_partial(_vp(xd), _vp(cd), _vp(sd), _vp(pd), per_seq, _vp(ck2), _vp(cv2), _vp(part), splits,
                                                b, h, kv, d, s_max, scale, 1, None, None, None, 0, None)
    lib.ternaspmm_attention_merge(_vp(part), splits, _vp(o2), b, h, d, None)
    torch.cuda.synchronize()
    assert torch.equal(ck1, ck2) and torch.equal(cv1, cv2)
    got = O.bf16_bits_to_f32(o2.cpu().numpy().view(np.uint16)).reshape(b, h, d).astype(np.float64)
    unsplit = O.bf16_bits_to_f32(o1.cpu().numpy().view(np.uint16)).reshape(b, h, d).astype(np.float64)
    tol = 2.0 ** -7 * np.abs(unsplit).max(axis=-1, keepdims=True) + 1e-6
    assert np.isfinite(got).all()
    assert (np.abs(got - unsplit) <= 2 * tol).all(), float((np.abs(got - unsplit) / tol).max())
    # the same launch with prefetching workgroups
    region = torch.zeros(40 * 2560, dtype=torch.int32, device="cuda")
    ptrs = (ctypes.c_void_p * 1)(region.data_ptr())
    sizes = (ctypes.c_longlong * 1)(region.numel() * 4)
    units = (ctypes.c_longlong * 1)(10240)
    part3 = _partial_buffer(lib, b, h, d)
    lib.ternaspmm_rope_decode_attention_partial(_vp(xd), _vp(cd), _vp(sd), _vp(pd), per_seq, _vp(ck3), _vp(cv3), _vp(part3), splits,
                                                b, h, kv, d, s_max, scale, 1, ptrs, sizes, units, 1, None)
    lib.ternaspmm_attention_merge(_vp(part3), splits, _vp(o3), b, h, d, None)
    torch.cuda.synchronize()
    assert torch.equal(o2, o3) and torch.equal(ck2, ck3) and torch.equal(cv2, cv3)


def test_attention_partial_against_the_oracle(lib):
    """Every sequence against attention_one_token at its own length, 8 splits over a 2B-shaped cache."""
    b, h, kv, d, s_max, lens = 2, 20, 5, 128, 1024, (1000, 333)
    qkv = make_bf16_activations(b, (h + 2 * kv) * d, 1811)
    k0 = make_bf16_activations(b * kv * s_max, d, 1812).reshape(b, kv, s_max, d)
    v0 = make_bf16_activations(b * kv * s_max, d, 1813, outlier_frac=0.01).reshape(b, kv, s_max, d)
    pos = np.array(lens, np.int64) - 1
    cos, sin = _angles(pos, d)
    xd, cd, sd, pd, ck, cv = _dev(qkv), _dev(cos), _dev(sin), _dev(pos), _dev(k0), _dev(v0)
    part = _partial_buffer(lib, b, h, d)
    out = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    lib.ternaspmm_rope_decode_attention_partial(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(ck), _vp(cv), _vp(part), 8,
                                                b, h, kv, d, s_max, float(d) ** -0.5, 1, None, None, None, 0, None)
    lib.ternaspmm_attention_merge(_vp(part), 8, _vp(out), b, h, d, None)
    torch.cuda.synchronize()
    got = O.bf16_bits_to_f32(out.cpu().numpy().view(np.uint16)).reshape(b, h, d).astype(np.float64)
    kc, vc = ck.cpu().numpy().view(np.uint16), cv.cpu().numpy().view(np.uint16)
    x = qkv.reshape(b, h + 2 * kv, d)
    for i in range(b):
        q = O.rope_adjacent(x[i:i + 1, :h], cos[i][None, None], sin[i][None, None])
        want = O.attention_one_token(q, kc[i:i + 1], vc[i:i + 1], lens[i], float(d) ** -0.5)[0]
        tol = 2.0 ** -7 * np.abs(want).max(axis=-1, keepdims=True) + 1e-6
        assert (np.abs(got[i] - want) <= tol).all(), (i, float((np.abs(got[i] - want) / tol).max()))
    assert lib.ternaspmm_attention_partial_splits(1, 20, 384) in (1, 2, 4, 8)
    assert lib.ternaspmm_attention_partial_splits(8, 20, 384) == 1


@pytest.mark.parametrize("splits", [1, 2, 4, 8])
@pytest.mark.parametrize("b,h,kv,d,s_max,lens", _random_attention_shapes(10, 20260903))
def test_attention_partial_random_shapes_against_the_oracle(lib, b, h, kv, d, s_max, lens, splits):
    """RoPE + cache write + split attention with the merge in a second launch, on shapes nobody tuned for (one
    workgroup per head or per kv head, whatever the library picks): every sequence against the oracle at its own length,
    the new cache rows against the oracle's rotation."""
    qkv = make_bf16_activations(b, (h + 2 * kv) * d, 1821 + b + s_max)
    k0 = make_bf16_activations(b * kv * s_max, d, 1822 + b).reshape(b, kv, s_max, d)
    v0 = make_bf16_activations(b * kv * s_max, d, 1823 + b, outlier_frac=0.01).reshape(b, kv, s_max, d)
    pos = np.array(lens, np.int64) - 1
    cos, sin = _angles(pos, d)
    xd, cd, sd, pd, ck, cv = _dev(qkv), _dev(cos), _dev(sin), _dev(pos), _dev(k0), _dev(v0)
    part = _partial_buffer(lib, b, h, d)
    out = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    print(f"[case] attention partial, random shape: b={b} h={h} kv={kv} d={d} S={s_max} lens={lens} splits={splits}", flush=True)
    lib.ternaspmm_rope_decode_attention_partial(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(ck), _vp(cv), _vp(part), splits,
                                                b, h, kv, d, s_max, float(d) ** -0.5, 1, None, None, None, 0, None)
    lib.ternaspmm_attention_merge(_vp(part), splits, _vp(out), b, h, d, None)
    torch.cuda.synchronize()
    got = O.bf16_bits_to_f32(out.cpu().numpy().view(np.uint16)).reshape(b, h, d).astype(np.float64)
    assert np.isfinite(got).all()
    kc, vc = ck.cpu().numpy().view(np.uint16), cv.cpu().numpy().view(np.uint16)
    x = qkv.reshape(b, h + 2 * kv, d)
    for i in range(b):
        c, sn = cos[i][None, None], sin[i][None, None]
        assert (kc[i][:, pos[i]] == O.rope_adjacent(x[i:i + 1, h:h + kv], c, sn)[0]).all() and (vc[i][:, pos[i]] == x[i, h + kv:]).all()
        untouched = np.setdiff1d(np.arange(s_max), pos[i])
        assert (kc[i][:, untouched] == k0[i][:, untouched]).all() and (vc[i][:, untouched] == v0[i][:, untouched]).all()
        want = O.attention_one_token(O.rope_adjacent(x[i:i + 1, :h], c, sn), kc[i:i + 1], vc[i:i + 1], lens[i], float(d) ** -0.5)[0]
        tol = 2.0 ** -7 * np.abs(want).max(axis=-1, keepdims=True) + 1e-6
        assert (np.abs(got[i] - want) <= tol).all(), (i, float((np.abs(got[i] - want) / tol).max()))


@pytest.mark.parametrize("splits", [1, 2, 4, 8])
@pytest.mark.parametrize("h,kv,d,n_out,s_max,n", [(20, 5, 128, 2560, 384, 300), (4, 2, 64, 320, 64, 5), (16, 8, 128, 1024, 1024, 1000)])
def test_fused_attention_merge_projection(lib, h, kv, d, n_out, s_max, n, splits):
    """bitlinear_TernaSpMM_packed_fused_attn (merge of the attention's partial results + sub-norm + quantisation +
    the O projection in one launch) against ternaspmm_attention_merge followed by bitlinear_TernaSpMM_packed_fused:
    output, published activations and scale bit-identical."""
    from tests.test_gpu_parity import repack
    from tests._util import DeviceFormat, make_ternary
    k_in = h * d
    w = make_ternary(n_out, k_in, 0.40, 1900 + h)
    packed = repack(lib, DeviceFormat(w))
    qkv = make_bf16_activations(1, (h + 2 * kv) * d, 1901 + n)
    k0 = make_bf16_activations(kv * s_max, d, 1902 + n).reshape(1, kv, s_max, d)
    v0 = make_bf16_activations(kv * s_max, d, 1903 + n, outlier_frac=0.01).reshape(1, kv, s_max, d)
    pos = np.array([n - 1], np.int64)
    cos, sin = _angles(pos, d)
    xd, cd, sd, pd, ck, cv = _dev(qkv), _dev(cos), _dev(sin), _dev(pos), _dev(k0), _dev(v0)
    part = _partial_buffer(lib, 1, h, d)
    lib.ternaspmm_rope_decode_attention_partial(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 0, _vp(ck), _vp(cv), _vp(part), splits,
                                                1, h, kv, d, s_max, float(d) ** -0.5, 1, None, None, None, 0, None)
    norm_w = _dev(make_bf16_activations(1, k_in, 1904).reshape(-1))
    ws = _dev(O.f32_to_bf16_bits(np.array([0.75, 0, 0, 0], np.float32)))
    # the pair
    attn = torch.zeros((1, k_in), dtype=torch.int16, device="cuda")
    out1 = torch.zeros((1, n_out), dtype=torch.int16, device="cuda")
    xq1, s1 = torch.zeros((1, k_in), dtype=torch.int8, device="cuda"), torch.zeros(1, dtype=torch.int16, device="cuda")
    lib.ternaspmm_attention_merge(_vp(part), splits, _vp(attn), 1, h, d, None)
    assert lib.bitlinear_TernaSpMM_packed_fused(_vp(attn), None, None, _vp(norm_w), 1e-5, _vp(packed), _vp(out1), _vp(ws), 1,
                                                _vp(xq1), _vp(s1), 1, n_out, k_in, None) == 1
    # one launch
    out2 = torch.zeros_like(out1)
    xq2, s2 = torch.zeros_like(xq1), torch.zeros_like(s1)
    print(f"[case] fused attention merge + O projection h={h} d={d} N={n_out} n={n} splits={splits}", flush=True)
    assert lib.bitlinear_TernaSpMM_packed_fused_attn(_vp(part), splits, d, _vp(norm_w), 1e-5, _vp(packed), _vp(out2), _vp(ws), 1,
                                                     _vp(xq2), _vp(s2), 1, n_out, k_in, None) == 1
    torch.cuda.synchronize()
    assert torch.equal(xq1, xq2) and torch.equal(s1, s2)
    assert torch.equal(out1, out2)
    assert int(xq2.abs().max().item()) >= 126                   # a real quantised row, not zeros
    # outside its range: two rows
    assert lib.bitlinear_TernaSpMM_packed_fused_attn(_vp(part), splits, d, _vp(norm_w), 1e-5, _vp(packed), _vp(out2), _vp(ws), 1,
                                                     None, None, 2, n_out, k_in, None) == 0


@pytest.mark.parametrize("splits", [1, 2, 4, 8])
@pytest.mark.parametrize("b,h,kv,d,s_max,lens", [(8, 20, 5, 128, 384, (300, 1, 129, 384, 77, 256, 200, 33)), (3, 4, 2, 64, 64, (5, 64, 17)),
                                                 (2, 16, 8, 128, 1024, (1000, 600))])
def test_attention_merge_rmsnorm_quant(lib, b, h, kv, d, s_max, lens, splits):
    """ternaspmm_attention_merge_rmsnorm_quant (merge of the splits + sub-norm + quantisation, one launch) against
    ternaspmm_attention_merge followed by ternaspmm_rmsnorm_quant: merged row, int8 values and scales bit-identical."""
    _merge_rmsnorm_quant_case(lib, b, h, kv, d, s_max, lens, splits)


@pytest.mark.parametrize("b,h,kv,d,s_max,lens,splits", [sh + (sp,) for sh, sp in zip(_random_attention_shapes(10, 20260907), [1, 2, 4, 8, 8, 4, 2, 1, 4, 8])])
def test_attention_merge_rmsnorm_quant_random_shapes(lib, b, h, kv, d, s_max, lens, splits):
    _merge_rmsnorm_quant_case(lib, b, h, kv, d, s_max, lens, splits)


def _merge_rmsnorm_quant_case(lib, b, h, kv, d, s_max, lens, splits):
    k_in = h * d
    qkv = make_bf16_activations(b, (h + 2 * kv) * d, 2100 + b)
    k0 = make_bf16_activations(b * kv * s_max, d, 2101 + b).reshape(b, kv, s_max, d)
    v0 = make_bf16_activations(b * kv * s_max, d, 2102 + b, outlier_frac=0.01).reshape(b, kv, s_max, d)
    pos = np.array(lens, np.int64).reshape(b, 1) - 1
    cos, sin = _angles(pos.reshape(-1), d)
    xd, cd, sd, pd, ck, cv = _dev(qkv), _dev(cos), _dev(sin), _dev(pos), _dev(k0), _dev(v0)
    part = _partial_buffer(lib, b, h, d)
    lib.ternaspmm_rope_decode_attention_partial(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(ck), _vp(cv), _vp(part), splits,
                                                b, h, kv, d, s_max, float(d) ** -0.5, 1, None, None, None, 0, None)
    norm_w = _dev(_weight(k_in, 2103))
    attn = torch.zeros((b, k_in), dtype=torch.int16, device="cuda")
    xq1, s1 = torch.zeros((b, k_in), dtype=torch.int8, device="cuda"), torch.zeros(b, dtype=torch.int16, device="cuda")
    lib.ternaspmm_attention_merge(_vp(part), splits, _vp(attn), b, h, d, None)
    lib.ternaspmm_rmsnorm_quant(_vp(attn), None, None, _vp(norm_w), 1e-5, None, _vp(xq1), _vp(s1), b, k_in, None)
    print(f"[case] attention merge + norm + quantise b={b} h={h} d={d} splits={splits}", flush=True)
    o2 = torch.zeros_like(attn)
    xq2, s2 = torch.zeros_like(xq1), torch.zeros_like(s1)
    if k_in > 4096:                                      # rows longer than the launch takes: declined, nothing enqueued
        assert lib.ternaspmm_attention_merge_rmsnorm_quant(_vp(part), splits, _vp(norm_w), 1e-5, _vp(o2), _vp(xq2), _vp(s2), b, h, d, None) == -1
        return
    assert lib.ternaspmm_attention_merge_rmsnorm_quant(_vp(part), splits, _vp(norm_w), 1e-5, _vp(o2), _vp(xq2), _vp(s2), b, h, d, None) == 0
    xq3, s3 = torch.zeros_like(xq1), torch.zeros_like(s1)
    assert lib.ternaspmm_attention_merge_rmsnorm_quant(_vp(part), splits, _vp(norm_w), 1e-5, None, _vp(xq3), _vp(s3), b, h, d, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(o2, attn) and torch.equal(xq2, xq1) and torch.equal(s2, s1)
    assert torch.equal(xq3, xq1) and torch.equal(s3, s1)
    assert int(xq2.abs().max().item()) >= 126
    # outside its range: nothing enqueued
    assert lib.ternaspmm_attention_merge_rmsnorm_quant(_vp(part), 3, _vp(norm_w), 1e-5, None, _vp(xq3), _vp(s3), b, h, d, None) == -1
    assert lib.ternaspmm_attention_merge_rmsnorm_quant(_vp(part), splits, _vp(norm_w), 1e-5, None, _vp(xq3), _vp(s3), b, 40, 128, None) == -1


@pytest.mark.parametrize("b,h,kv,d,s_max,lens", [(8, 20, 5, 128, 384, (300, 1, 129, 384, 77, 256, 200, 33)), (3, 4, 2, 64, 64, (5, 64, 17)),
                                                 (12, 20, 5, 128, 256, tuple(range(20, 260, 20)))])
def test_rope_decode_attention_with_norm_statistics(lib, b, h, kv, d, s_max, lens):
    """ternaspmm_rope_decode_attention_stats: the output row and the caches are those of ternaspmm_rope_decode_attention
    (no workspace: the unsplit launch); the statistics are, per sequence and head, the sum of squares (fp32 accuracy) and
    the exact max |o * w| of the stored bf16 row; ternaspmm_quant_from_stats on them agrees with the norm kernel's scales
    up to one bf16 step."""
    k_in = h * d
    qkv = make_bf16_activations(b, (h + 2 * kv) * d, 2200 + b)
    k0 = make_bf16_activations(b * kv * s_max, d, 2201 + b).reshape(b, kv, s_max, d)
    v0 = make_bf16_activations(b * kv * s_max, d, 2202 + b, outlier_frac=0.01).reshape(b, kv, s_max, d)
    pos = np.array(lens, np.int64).reshape(b, 1) - 1
    cos, sin = _angles(pos.reshape(-1), d)
    w = _weight(k_in, 2203)
    xd, cd, sd, pd, wd = _dev(qkv), _dev(cos), _dev(sin), _dev(pos), _dev(w)
    ck1, cv1, ck2, cv2 = _dev(k0), _dev(v0), _dev(k0), _dev(v0)
    o1 = torch.zeros((b, k_in), dtype=torch.int16, device="cuda")
    o2 = torch.zeros_like(o1)
    st = torch.full((b, h, 2), float("nan"), dtype=torch.float32, device="cuda")
    print(f"[case] attention with norm statistics b={b} h={h} d={d}", flush=True)
    lib.ternaspmm_rope_decode_attention(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(ck1), _vp(cv1), _vp(o1), b, h, kv, d, s_max,
                                        float(d) ** -0.5, 1, None, None)
    assert lib.ternaspmm_rope_decode_attention_stats(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(ck2), _vp(cv2), _vp(o2), b, h, kv, d, s_max,
                                                     float(d) ** -0.5, 1, _vp(wd), _vp(st), None) == h
    torch.cuda.synchronize()
    assert torch.equal(o1, o2) and torch.equal(ck1, ck2) and torch.equal(cv1, cv2)
    o = O.bf16_bits_to_f32(o2.cpu().numpy().view(np.uint16)).reshape(b, h, d)
    wf = O.bf16_bits_to_f32(w).reshape(1, h, d)
    got = st.cpu().numpy()
    assert (got[:, :, 1] == np.abs(o * wf).max(axis=2)).all()
    assert np.allclose(got[:, :, 0], (o.astype(np.float64) ** 2).sum(axis=2), rtol=2e-6, atol=1e-30)
    # the consumer: quantised rows from these partials against the norm kernel on the same row
    xq1, s1 = torch.zeros((b, k_in), dtype=torch.int8, device="cuda"), torch.zeros(b, dtype=torch.int16, device="cuda")
    xq2, s2 = torch.zeros_like(xq1), torch.zeros_like(s1)
    lib.ternaspmm_rmsnorm_quant(_vp(o2), None, None, _vp(wd), 1e-5, None, _vp(xq1), _vp(s1), b, k_in, None)
    assert lib.ternaspmm_quant_from_stats(_vp(o2), _vp(st), h, _vp(wd), 1e-5, _vp(xq2), _vp(s2), b, k_in, None) == 0
    torch.cuda.synchronize()
    assert np.abs(_bf16_key(s1.cpu().numpy().view(np.uint16)) - _bf16_key(s2.cpu().numpy().view(np.uint16))).max() <= 1
    same = (s1 == s2).cpu().numpy()
    dq = np.abs(xq1.cpu().numpy().astype(np.int32) - xq2.cpu().numpy().astype(np.int32))[same]
    assert dq.size and dq.max() <= 1 and (dq != 0).mean() < 0.02
    assert lib.ternaspmm_rope_decode_attention_stats(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(ck2), _vp(cv2), _vp(o2), b, h, kv, d, s_max,
                                                     float(d) ** -0.5, 1, None, _vp(st), None) == -1


@pytest.mark.parametrize("splits", [1, 4])
@pytest.mark.parametrize("b,h,kv,d,s_max,n", [(2, 4, 2, 64, 300, 17), (8, 20, 5, 128, 384, 300), (2, 16, 8, 128, 100, 77), (1, 20, 5, 128, 384, 200)])
def test_rope_decode_attention_partial_rotate_half(lib, b, h, kv, d, s_max, n, splits):
    """The deferred-merge launches with the rotate-half pairing of RoPE (adjacent = 0; several sequences with 2 or 4 heads
    per kv head run one workgroup per kv head): caches bit-identical to ternaspmm_rope_decode_attention, merged output
    within the attention tolerance of the unsplit launch."""
    lens = [max(1, n - 5 * i) for i in range(b)]
    qkv = make_bf16_activations(b, (h + 2 * kv) * d, 2301 + n)
    k0 = make_bf16_activations(b * kv * s_max, d, 2302 + n).reshape(b, kv, s_max, d)
    v0 = make_bf16_activations(b * kv * s_max, d, 2303 + n, outlier_frac=0.01).reshape(b, kv, s_max, d)
    pos = np.array(lens, np.int64) - 1
    cos, sin = _angles(pos, d)
    xd, cd, sd, pd = _dev(qkv), _dev(cos), _dev(sin), _dev(pos)
    scale = float(d) ** -0.5
    ck1, cv1, ck2, cv2 = _dev(k0), _dev(v0), _dev(k0), _dev(v0)
    o1 = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    o2 = torch.zeros_like(o1)
    print(f"[case] attention partial + merge, rotate-half b={b} h={h} kv={kv} d={d} n={n} splits={splits}", flush=True)
    lib.ternaspmm_rope_decode_attention(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(ck1), _vp(cv1), _vp(o1), b, h, kv, d, s_max,
                                        scale, 0, None, None)
    part = _partial_buffer(lib, b, h, d)
    lib.ternaspmm_rope_decode_attention_partial(_vp(xd), _vp(cd), _vp(sd), _vp(pd), 1, _vp(ck2), _vp(cv2), _vp(part), splits,
                                                b, h, kv, d, s_max, scale, 0, None, None, None, 0, None)
    lib.ternaspmm_attention_merge(_vp(part), splits, _vp(o2), b, h, d, None)
    torch.cuda.synchronize()
    assert torch.equal(ck1, ck2) and torch.equal(cv1, cv2)
    got = O.bf16_bits_to_f32(o2.cpu().numpy().view(np.uint16)).reshape(b, h, d).astype(np.float64)
    unsplit = O.bf16_bits_to_f32(o1.cpu().numpy().view(np.uint16)).reshape(b, h, d).astype(np.float64)
    tol = 2.0 ** -7 * np.abs(unsplit).max(axis=-1, keepdims=True) + 1e-6
    assert np.isfinite(got).all()
    assert (np.abs(got - unsplit) <= 2 * tol).all(), float((np.abs(got - unsplit) / tol).max())
