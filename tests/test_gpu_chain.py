"""GPU tests of the chained small-M linears (ternaspmm_fused_linear, ternaspmm_row_stats, ternaspmm_interleave_gate_up)
through the C ABI, against the CPU oracle.

Bars, as for the other prologue kernels: everything whose arithmetic is fully defined is bit-exact -- the residual
stream, the gate, the integer matmul + epilogue on the (xq, s) the launch publishes, the partial maxima (products of
two bf16 values are exact in fp32); sums of squares to fp32 summation accuracy; the norm output, which no launch
publishes, through its consequences: s within one bf16 step of the float64 evaluation's, xq within one step on rows
whose scale agrees, max |xq| of every row at 126 or 127 (the scale really is that of the row's largest |y|)."""
import numpy as np
import pytest
import torch

import ternainfer_amd as T
from ternainfer_amd import linear as L
from oracle import terna_oracle as O
from tests._util import DeviceFormat, make_bf16_activations, make_ternary

pytestmark = pytest.mark.gpu


def _bf(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda().view(torch.bfloat16)


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _key(b):
    b = b.astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)


def _weight(k, seed):
    return O.f32_to_bf16_bits(np.random.default_rng(seed).uniform(0.5, 1.5, k).astype(np.float32))


def _packed(w):
    fmt = DeviceFormat(w)
    p = T.repack_weight(fmt.vals, fmt.off, fmt.med, fmt.bm, *w.shape)
    torch.cuda.synchronize()
    return p


WS = O.f32_to_bf16_bits(np.array([1.25, 0.75, 1.5, 0.0], np.float32))


def _check_quantiser(h_bits, g_bits, q, s, eps=1e-5):
    """(xq, s) as published against the float64 norm of h: see the module header."""
    y64 = O.rmsnorm(h_bits, g_bits, eps)
    q_ref, s_ref = O.quant_input(y64)
    assert np.abs(_key(s) - _key(s_ref)).max() <= 1
    same = s == s_ref
    dq = np.abs(q.astype(np.int32) - q_ref.astype(np.int32))[same]
    assert dq.size and dq.max() <= 1 and (dq != 0).mean() < 0.02
    assert set(np.abs(q.astype(np.int32)).max(axis=1).tolist()) <= {126, 127}


def _check_stats(stats, h_bits, next_w_bits, width):
    """Partials over `width` columns each: maxima exact, sums of squares to fp32 accuracy."""
    h = O.bf16_bits_to_f32(h_bits)
    m, k = h.shape
    count = -(-k // width)
    pad = count * width - k
    hp = np.pad(h, ((0, 0), (0, pad))).reshape(m, count, width)
    wp = np.pad(O.bf16_bits_to_f32(next_w_bits), (0, pad)).reshape(1, count, width)
    assert stats.shape == (m, count, 2)
    assert (stats[:, :, 1] == np.abs(hp * wp).max(axis=2)).all()
    want = (hp.astype(np.float64) ** 2).sum(axis=2)
    assert np.allclose(stats[:, :, 0], want, rtol=2e-6, atol=1e-30)


@pytest.mark.parametrize("m,k", [(1, 2560), (8, 2560), (3, 6912), (5, 520), (2, 64)])
def test_row_stats(m, k):
    h = make_bf16_activations(m, k, 1200 + m + k, outlier_frac=0.01)
    g = _weight(k, 1201 + k)
    print(f"[case] row stats m={m} k={k}", flush=True)
    st = L.row_stats(_bf(h), _bf(g)).cpu().numpy()
    _check_stats(st, h, g, 512)


@pytest.mark.parametrize("b,v,k,s_len,half,per_seq", [(1, 128256, 2560, 384, 64, False), (8, 128256, 2560, 384, 64, False),
                                                       (5, 1000, 520, 40, 32, True), (16, 300, 64, 2048, 64, True), (3, 50, 6912, 7, 4, True)])
def test_step_inputs(b, v, k, s_len, half, per_seq):
    """ternaspmm_step_inputs against the three launches it stands for: the embedding rows (bit copies), their partials
    exactly as ternaspmm_row_stats leaves them, the RoPE-table rows of the positions (shared or per sequence)."""
    gen = torch.Generator().manual_seed(1300 + b + k)
    emb = (torch.randn((v, k), generator=gen) * 0.02).to(torch.bfloat16).cuda()
    table = torch.randn((s_len, 2, half), generator=gen).cuda()
    g = _weight(k, 1301 + k)
    tokens = torch.randint(0, v, (b, 1), generator=gen).cuda()
    tokens[0, 0] = v - 1
    pos = torch.randint(0, s_len, (b if per_seq else 1,), generator=gen).cuda()
    pos[-1] = s_len - 1
    print(f"[case] step inputs b={b} v={v} k={k} S={s_len} half={half} per_seq={per_seq}", flush=True)
    x, stats, cos, sin = L.step_inputs(tokens, pos, emb, table, _bf(g))
    torch.cuda.synchronize()
    want = emb[tokens.reshape(-1)]
    assert torch.equal(x, want)
    assert torch.equal(stats, L.row_stats(want, _bf(g)))
    rows = table.index_select(0, pos.expand(b) if not per_seq else pos)
    assert torch.equal(cos, rows[:, 0]) and torch.equal(sin, rows[:, 1])
    assert cos.is_contiguous() and sin.is_contiguous()


def test_step_inputs_clamps_and_refuses():
    """Tokens and positions come from device memory the host cannot check: values outside their tables are clamped, not
    followed.  Shapes and pointers the kernel cannot take are refused on the host (-1, nothing launched)."""
    import ctypes
    from ternainfer_amd import _lib
    lib = _lib.load()
    v, k, s_len, half = 40, 128, 16, 8
    emb = (torch.randn((v, k)) * 0.02).to(torch.bfloat16).cuda()
    table = torch.randn((s_len, 2, half)).cuda()
    g = _bf(_weight(k, 1310))
    tokens = torch.tensor([[-5], [v + 100], [7]], dtype=torch.int64).cuda()
    pos = torch.tensor([s_len + 3, -1, 2], dtype=torch.int64).cuda()
    x, stats, cos, sin = L.step_inputs(tokens, pos, emb, table, g)
    torch.cuda.synchronize()
    assert torch.equal(x, emb[torch.tensor([0, v - 1, 7]).cuda()])
    assert torch.equal(cos, table[torch.tensor([s_len - 1, 0, 2]).cuda(), 0]) and torch.equal(sin, table[torch.tensor([s_len - 1, 0, 2]).cuda(), 1])
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    xo, so, ro = torch.empty_like(x), torch.empty_like(stats), torch.empty((2, 3, half), device="cuda")
    ok = lambda **kw: lib.ternaspmm_step_inputs(p(tokens), p(pos), 1, kw.get("emb", p(emb)), v, kw.get("k", k), p(table), s_len, kw.get("half", half),
                                                p(g), p(xo), p(so), kw.get("rope", p(ro)), kw.get("b", 3), None)
    assert ok() == 1
    assert ok(k=124) == -1 and ok(half=6) == -1 and ok(b=0) == -1 and ok(emb=None) == -1
    assert ok(rope=ctypes.c_void_p(ro.data_ptr() + 4)) == -1
    torch.cuda.synchronize()


@pytest.mark.parametrize("m", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("n,k,ws_num", [(3840, 2560, 3), (2560, 2560, 1), (2560, 6912, 1), (256, 192, 2)])
def test_stats_prologue_with_store_and_residual_epilogues(m, n, k, ws_num):
    _stats_prologue_case(m, n, k, ws_num)


def _random_chain_shapes(count, seed):
    """Seeded shapes nobody tuned for: 1 - 8 rows, N and K any multiple of 64 (K up to 112 k-tiles, the longest the
    statistics-given kernels take), weight-scale groups that divide N."""
    rng = np.random.default_rng(seed)
    shapes = []
    for _ in range(count):
        n = 64 * int(rng.integers(1, 33))
        k = 64 * int(rng.choice([rng.integers(1, 13), rng.integers(13, 41), rng.integers(41, 113)]))
        shapes.append((int(rng.integers(1, 9)), n, k, int(rng.choice([g for g in (1, 2, 3, 4) if n % g == 0]))))
    return shapes


@pytest.mark.parametrize("m,n,k,ws_num", _random_chain_shapes(16, 20260901))
def test_stats_prologue_random_shapes(m, n, k, ws_num):
    _stats_prologue_case(m, n, k, ws_num)


def _stats_prologue_case(m, n, k, ws_num):
    w = make_ternary(n, k, 0.40, 1210 + m + n)
    packed = _packed(w)
    h = make_bf16_activations(m, k, 1211 + m + k, outlier_frac=0.01)
    g = _weight(k, 1212 + k)
    nxt = _weight(n, 1213 + n)
    res = make_bf16_activations(m, n, 1214 + m + n)
    ws = _bf(WS)
    stats = L.row_stats(_bf(h), _bf(g))
    print(f"[case] chain linear, statistics given: m={m} n={n} k={k} ws_num={ws_num}", flush=True)
    r = L.fused_linear(_bf(h), _bf(g), 1e-5, packed, ws, ws_num, n, k, stats=stats, publish=True)
    assert r is not None
    out, st_out, raw, xq, s = r
    torch.cuda.synchronize()
    q, sb = xq.cpu().numpy(), _bits(s)
    _check_quantiser(h, g, q, sb)
    want = O.spmm_i8(q, w, sb, WS, ws_num, 0)
    assert (_bits(out) == want).all() and st_out is None and raw is None
    # the same launch as a producer: the stream after this linear and its statistics under the next norm
    r = L.fused_linear(_bf(h), _bf(g), 1e-5, packed, ws, ws_num, n, k, stats=stats, epilogue=L.EPILOGUE_RESIDUAL,
                       residual=_bf(res), next_norm_weight=_bf(nxt), want_raw=True, publish=True)
    out2, st_out, raw, xq2, s2 = r
    torch.cuda.synchronize()
    assert torch.equal(xq2, xq) and torch.equal(s2, s)
    assert (_bits(raw) == want).all()
    h_next = O.residual_add(res, want)
    assert (_bits(out2) == h_next).all()
    _check_stats(st_out.cpu().numpy(), h_next, nxt, 16)
    # ... and the consumer of THAT: statistics from the producing epilogue, not from ternaspmm_row_stats
    if n <= 2560:
        w2 = make_ternary(256, n, 0.40, 1215 + m)
        p2 = _packed(w2)
        r = L.fused_linear(out2, _bf(nxt), 1e-5, p2, ws, 1, 256, n, stats=st_out, publish=True)
        out3, _, _, xq3, s3 = r
        torch.cuda.synchronize()
        _check_quantiser(h_next, nxt, xq3.cpu().numpy(), _bits(s3))
        assert (_bits(out3) == O.spmm_i8(xq3.cpu().numpy(), w2, _bits(s3), WS, 1, 0)).all()


@pytest.mark.parametrize("m", [1, 2, 4, 8])
@pytest.mark.parametrize("f,k", [(6912, 2560), (128, 192)])
def test_gate_epilogue_on_interleaved_gate_up(m, f, k):
    """gate+up with the bands of w1 and w3 interleaved at load time: inner = relu(x1)^2 * x3 leaves the launch, x13 never
    exists in memory.  The oracle works on the ordinary [w1; w3] matrix."""
    n = 2 * f
    w13 = make_ternary(n, k, 0.40, 1220 + m + f)
    plain = _packed(w13)
    inter = L.interleave_gate_up(plain, n, k)
    torch.cuda.synchronize()
    # the permutation itself: band 2j <- band j, band 2j+1 <- band f/16 + j
    a = plain.view(n // 16, -1).cpu()
    b = inter.view(n // 16, -1).cpu()
    assert torch.equal(b[0::2], a[: f // 16]) and torch.equal(b[1::2], a[f // 16:])
    h = make_bf16_activations(m, k, 1221 + m + k, outlier_frac=0.01)
    g = _weight(k, 1222 + k)
    nxt = _weight(f, 1223 + f)
    stats = L.row_stats(_bf(h), _bf(g))
    print(f"[case] chain gate+up: m={m} f={f} k={k}", flush=True)
    r = L.fused_linear(_bf(h), _bf(g), 1e-5, inter, _bf(WS), 2, n, k, stats=stats, epilogue=L.EPILOGUE_GATE,
                       next_norm_weight=_bf(nxt), publish=True)
    assert r is not None
    inner, st_out, _, xq, s = r
    torch.cuda.synchronize()
    q, sb = xq.cpu().numpy(), _bits(s)
    _check_quantiser(h, g, q, sb)
    x13 = O.spmm_i8(q, w13, sb, WS, 2, 0)
    want = O.relu2_mul(x13)
    assert inner.shape == (m, f) and (_bits(inner) == want).all()
    _check_stats(st_out.cpu().numpy(), want, nxt, 16)
    # the same launch fed with activations that are quantised already: the same bits
    print(f"[case] chain gate+up, quantised activations: m={m} f={f} k={k}", flush=True)
    r = L.fused_linear(xq, None, 1e-5, inter, _bf(WS), 2, n, k, quantised=s, epilogue=L.EPILOGUE_GATE, next_norm_weight=_bf(nxt))
    assert r is not None
    torch.cuda.synchronize()
    assert torch.equal(r[0], inner) and torch.equal(r[1], st_out)


@pytest.mark.parametrize("m", [9, 11, 16])
@pytest.mark.parametrize("f,k", [(6912, 2560), (128, 192), (64, 6144)])
def test_gate_epilogue_on_quantised_rows_above_eight(m, f, k):
    """The gate epilogue fed with quantised rows takes up to 16 of them (the statistics-fed prologue stops at 8): the norm
    kernel's (xq, s) in, relu(x1)^2 * x3 and its partials out, against the oracle on the ordinary [w1; w3] matrix."""
    n = 2 * f
    w13 = make_ternary(n, k, 0.40, 1270 + m + f)
    inter = L.interleave_gate_up(_packed(w13), n, k)
    h = make_bf16_activations(m, k, 1271 + m + k, outlier_frac=0.01)
    g, nxt = _weight(k, 1272 + k), _weight(f, 1273 + f)
    xq, s, _ = L.rmsnorm_quant(_bf(h), _bf(g), 1e-5)
    print(f"[case] chain gate+up, quantised activations: m={m} f={f} k={k}", flush=True)
    r = L.fused_linear(xq, None, 1e-5, inter, _bf(WS), 2, n, k, quantised=s, epilogue=L.EPILOGUE_GATE, next_norm_weight=_bf(nxt))
    assert r is not None
    torch.cuda.synchronize()
    want = O.relu2_mul(O.spmm_i8(xq.cpu().numpy(), w13, _bits(s), WS, 2, 0))
    assert r[0].shape == (m, f) and (_bits(r[0]) == want).all()
    _check_stats(r[1].cpu().numpy(), want, nxt, 16)


def test_norm_and_attention_prologues_with_the_residual_epilogue():
    """The prologues that take their statistics inside, now with the producing epilogue: the raw output must be the
    bits of the existing entry points (same kernel arithmetic), the stream their residual sum."""
    lib = T._lib.load()
    n = k = 2560
    w = make_ternary(n, k, 0.40, 1230)
    packed = _packed(w)
    g, nxt = _weight(k, 1231), _weight(n, 1232)
    ws = _bf(WS)
    for m in (2, 8):
        h = make_bf16_activations(m, k, 1233 + m)
        res = make_bf16_activations(m, n, 1234 + m)
        print(f"[case] chain linear, statistics inside + residual epilogue: m={m}", flush=True)
        r = L.fused_linear(_bf(h), _bf(g), 1e-5, packed, ws, 1, n, k, epilogue=L.EPILOGUE_RESIDUAL, residual=_bf(res),
                           next_norm_weight=_bf(nxt), want_raw=True, publish=True)
        out, st, raw, xq, s = r
        old, _ = T.rmsnorm_linear_packed(_bf(h), _bf(g), 1e-5, packed, ws, 1, n) if m <= 8 else (None, None)
        torch.cuda.synchronize()
        assert torch.equal(raw, old)
        h_next = O.residual_add(res, _bits(raw))
        assert (_bits(out) == h_next).all()
        _check_stats(st.cpu().numpy(), h_next, nxt, 16)
        assert (_bits(raw) == O.spmm_i8(xq.cpu().numpy(), w, _bits(s), WS, 1, 0)).all()
    # attention partials -> merge inside -> O projection -> residual epilogue (one sequence)
    heads, hd, splits = 20, 128, 4
    nbytes = lib.ternaspmm_attention_partial_bytes(1, heads, hd)
    rng = np.random.default_rng(1240)
    part = torch.from_numpy(rng.standard_normal(nbytes // 4).astype(np.float32)).cuda()
    stat_floats = nbytes // 4 - heads * 8 * hd
    # statistics block: maxima then sums of numerators per head and split -- keep the sums positive
    part[:stat_floats] = part[:stat_floats].abs() + 0.5
    res = make_bf16_activations(1, n, 1241)
    print("[case] chain linear, attention merge inside + residual epilogue", flush=True)
    old = T.linear.attention_merge_rmsnorm_linear_packed(part, splits, heads, hd, _bf(g), 1e-5, packed, ws, 1, n)
    r = L.fused_linear(part, _bf(g), 1e-5, packed, ws, 1, n, k, attention=(splits, hd), epilogue=L.EPILOGUE_RESIDUAL,
                       residual=_bf(res), next_norm_weight=_bf(nxt), want_raw=True)
    out, st, raw, _, _ = r
    torch.cuda.synchronize()
    assert torch.equal(raw, old)
    h_next = O.residual_add(res, _bits(raw))
    assert (_bits(out) == h_next).all()
    _check_stats(st.cpu().numpy(), h_next, nxt, 16)


@pytest.mark.parametrize("m", [1, 5, 8, 11, 16])
@pytest.mark.parametrize("n,k", [(2560, 6912), (2560, 2560), (8256, 192)])
def test_quantise_launch_and_quantised_prologue(m, n, k):
    """The norm + quantisation as a launch of its own from the producer's partials, and the small-M linear on its output
    with the producing epilogue: (xq, s) must be the bits the statistics-fed prologue forms inside its launch (up to 8
    rows, where both exist), the linear exact on them, the stream and its partials as for the other producers."""
    w = make_ternary(n, k, 0.40, 1260 + m + n)
    packed = _packed(w)
    h = make_bf16_activations(m, k, 1261 + m + k, outlier_frac=0.01)
    g, nxt = _weight(k, 1262 + k), _weight(n, 1263 + n)
    res = make_bf16_activations(m, n, 1264 + m + n)
    ws = _bf(WS)
    stats = L.row_stats(_bf(h), _bf(g))
    print(f"[case] quantise launch + quantised prologue: m={m} n={n} k={k}", flush=True)
    xq, s = L.quant_from_stats(_bf(h), stats, _bf(g), 1e-5)
    torch.cuda.synchronize()
    q, sb = xq.cpu().numpy(), _bits(s)
    _check_quantiser(h, g, q, sb)
    if m <= 8 and n <= 2560:
        r = L.fused_linear(_bf(h), _bf(g), 1e-5, packed, ws, 1, n, k, stats=stats, publish=True)
        assert torch.equal(r[3], xq) and torch.equal(r[4], s)
    r = L.fused_linear(xq, None, 1e-5, packed, ws, 1, n, k, quantised=s, epilogue=L.EPILOGUE_RESIDUAL, residual=_bf(res),
                       next_norm_weight=_bf(nxt), want_raw=True)
    if n // 16 > 448:
        assert r is None                                   # more partials per row than a consumer adds up
        return
    out, st, raw, _, _ = r
    torch.cuda.synchronize()
    want = O.spmm_i8(q, w, sb, WS, 1, 0)
    assert (_bits(raw) == want).all()
    h_next = O.residual_add(res, want)
    assert (_bits(out) == h_next).all()
    _check_stats(st.cpu().numpy(), h_next, nxt, 16)


def _random_quantised_shapes(count, seed, gate):
    """Seeded shapes for the linears on quantised rows: 1 - 16 rows, N any multiple of 64 (gate: F any multiple of 32, N = 2 F),
    K any multiple of 64 up to what the epilogue takes (gate: 6144)."""
    rng = np.random.default_rng(seed)
    shapes = []
    for _ in range(count):
        m = int(rng.choice([rng.integers(1, 9), rng.integers(9, 17)]))
        k = 64 * int(rng.choice([rng.integers(1, 13), rng.integers(13, 97 if gate else 113)]))
        shapes.append((m, 32 * int(rng.integers(1, 65)) if gate else 64 * int(rng.integers(1, 41)), k))
    return shapes


@pytest.mark.parametrize("m,n,k", _random_quantised_shapes(12, 20260905, False))
def test_quantised_prologue_residual_random_shapes(m, n, k):
    """ternaspmm_quant_from_stats + the linear on its rows with the residual epilogue, on shapes nobody tuned for: the
    integers exact on the published (xq, s), the stream and the partials of the next norm as for the other producers."""
    w = make_ternary(n, k, 0.40, 1280 + m + n)
    packed = _packed(w)
    h = make_bf16_activations(m, k, 1281 + m + k, outlier_frac=0.01)
    g, nxt = _weight(k, 1282 + k), _weight(n, 1283 + n)
    res = make_bf16_activations(m, n, 1284 + m + n)
    xq, s = L.quant_from_stats(_bf(h), L.row_stats(_bf(h), _bf(g)), _bf(g), 1e-5)
    print(f"[case] quantised prologue, residual epilogue, random shape: m={m} n={n} k={k}", flush=True)
    r = L.fused_linear(xq, None, 1e-5, packed, _bf(WS), 1, n, k, quantised=s, epilogue=L.EPILOGUE_RESIDUAL, residual=_bf(res),
                       next_norm_weight=_bf(nxt), want_raw=True)
    assert r is not None
    out, st, raw, _, _ = r
    torch.cuda.synchronize()
    q, sb = xq.cpu().numpy(), _bits(s)
    _check_quantiser(h, g, q, sb)
    want = O.spmm_i8(q, w, sb, WS, 1, 0)
    assert (_bits(raw) == want).all()
    h_next = O.residual_add(res, want)
    assert (_bits(out) == h_next).all()
    _check_stats(st.cpu().numpy(), h_next, nxt, 16)


@pytest.mark.parametrize("m,f,k", _random_quantised_shapes(12, 20260906, True))
def test_quantised_prologue_gate_random_shapes(m, f, k):
    n = 2 * f
    w13 = make_ternary(n, k, 0.40, 1290 + m + f)
    inter = L.interleave_gate_up(_packed(w13), n, k)
    h = make_bf16_activations(m, k, 1291 + m + k, outlier_frac=0.01)
    g, nxt = _weight(k, 1292 + k), _weight(f, 1293 + f)
    xq, s, _ = L.rmsnorm_quant(_bf(h), _bf(g), 1e-5)
    print(f"[case] quantised prologue, gate epilogue, random shape: m={m} f={f} k={k}", flush=True)
    r = L.fused_linear(xq, None, 1e-5, inter, _bf(WS), 2, n, k, quantised=s, epilogue=L.EPILOGUE_GATE, next_norm_weight=_bf(nxt))
    assert r is not None
    torch.cuda.synchronize()
    want = O.relu2_mul(O.spmm_i8(xq.cpu().numpy(), w13, _bits(s), WS, 2, 0))
    assert r[0].shape == (m, f) and (_bits(r[0]) == want).all()
    _check_stats(r[1].cpu().numpy(), want, nxt, 16)


def test_unsupported_combinations_are_declined():
    n, k = 256, 192
    packed = _packed(make_ternary(n, k, 0.4, 1250))
    h, g = _bf(make_bf16_activations(9, k, 1251)), _bf(_weight(k, 1252))
    assert L.fused_linear(h, g, 1e-5, packed, _bf(WS), 1, n, k, stats=L.row_stats(h, g)) is None          # M > 8
    h = h[:2].contiguous()
    assert L.fused_linear(h, g, 1e-5, packed, _bf(WS), 1, n, k) is None                                    # NORM + STORE: the older entry point
    assert L.fused_linear(h, g, 1e-5, packed, _bf(WS), 1, n, k, stats=L.row_stats(h, g), epilogue=L.EPILOGUE_GATE,
                          next_norm_weight=_bf(_weight(n // 2, 1253))) is None                              # GATE needs two scale groups
    xq9 = torch.zeros((17, k), dtype=torch.int8, device="cuda")
    s9 = torch.ones(17, dtype=torch.bfloat16, device="cuda")
    assert L.fused_linear(xq9, None, 1e-5, packed, _bf(WS), 2, n, k, quantised=s9, epilogue=L.EPILOGUE_GATE,
                          next_norm_weight=_bf(_weight(n // 2, 1254))) is None                              # GATE on quantised rows: up to 16
    assert L.fused_linear(xq9, None, 1e-5, packed, _bf(WS), 1, n, k, quantised=s9) is None                 # QUANTISED + STORE: bitlinear_TernaSpMM_packed
    torch.cuda.synchronize()
