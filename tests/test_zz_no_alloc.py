"""ternaspmm_decode_attention_static: the entry point that allocates nothing (its split-attention scratch is a
static device array inside the library) against ternaspmm_decode_attention with a caller workspace -- same
kernels, same split order, so the outputs must be identical bit for bit -- on two calls in a row, the second
with a smaller input, then a third that is larger again (the counters sit at a fixed place and every launch
leaves them at zero).  Collected last: it shares the library's one scratch array with nothing else."""
import ctypes

import numpy as np
import pytest
import torch

from tests._util import make_bf16_activations

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(a.view(np.int16) if a.dtype == np.uint16 else a).cuda()


def _vp(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _inputs(b, h, kv, d, s_max, n, seed):
    """`n`: the prefix length shared by the batch, or one length per sequence (-> per_sequence = 1)."""
    q = make_bf16_activations(b * h, d, seed).reshape(b, h, d)
    k = make_bf16_activations(b * kv * s_max, d, seed + 1).reshape(b, kv, s_max, d)
    v = make_bf16_activations(b * kv * s_max, d, seed + 2, outlier_frac=0.01).reshape(b, kv, s_max, d)
    per_seq = int(not isinstance(n, int))
    pos = np.array([n - 1] if not per_seq else [x - 1 for x in n], np.int64)
    return _dev(q), _dev(k), _dev(v), _dev(pos), per_seq


def _case(lib, b, h, kv, d, s_max, n, seed):
    qd, kd, vd, pd, per_seq = _inputs(b, h, kv, d, s_max, n, seed)
    scale = float(d) ** -0.5
    ws = torch.zeros(lib.ternaspmm_attention_workspace_bytes(b, h, d), dtype=torch.int8, device="cuda")
    want = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    lib.ternaspmm_decode_attention(_vp(qd), _vp(kd), _vp(vd), _vp(pd), per_seq, _vp(want), b, h, kv, d, s_max, scale, _vp(ws), None)
    got = torch.full((b, h * d), -1, dtype=torch.int16, device="cuda")
    print(f"[case] decode attention, static scratch: b={b} h={h} kv={kv} d={d} S={s_max} n={n}", flush=True)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]                      # device memory as the driver sees it
    rc = lib.ternaspmm_decode_attention_static(_vp(qd), _vp(kd), _vp(vd), _vp(pd), per_seq, _vp(got), b, h, kv, d, s_max, scale, None)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the amount of free device memory"
    assert rc == 0
    assert torch.equal(got, want), f"static-scratch output differs (b={b} h={h} S={s_max} n={n})"
    assert int(want.abs().sum().item()) != 0


def test_static_scratch_first_call_under_capture_is_refused(capfd):
    """Runs first in this file (in a fresh process the array has not been set up yet; after other tests that used the
    entry point the call is simply recorded, which is as valid): the set-up clear must not end up inside a graph."""
    from ternainfer_amd import _lib
    lib = _lib.load()
    b, h, kv, d, s_max = 1, 20, 5, 128, 1024
    qd, kd, vd, pd, _ = _inputs(b, h, kv, d, s_max, 900, 9000)
    out = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.ternaspmm_decode_attention_static(_vp(qd), _vp(kd), _vp(vd), _vp(pd), 0, _vp(out), b, h, kv, d, s_max,
                                                       float(d) ** -0.5, ctypes.c_void_p(side.cuda_stream))
    err = capfd.readouterr().err
    assert (rc == -1 and "outside stream capture" in err) or rc == 0
    del graph
    torch.cuda.synchronize()


def test_static_scratch_entry_point_matches_the_workspace_one():
    from ternainfer_amd import _lib
    lib = _lib.load()
    assert torch.cuda.is_available()
    # caches of >= 1024 slots: the prefix of every head is split over several workgroups, so the scratch is in use
    _case(lib, 8, 20, 5, 128, 1024, 1000, 9100)        # 160 heads
    _case(lib, 1, 20, 5, 128, 2048, 1500, 9200)        # smaller: 20 heads, 8 splits
    _case(lib, 2, 4, 2, 64, 1040, 1030, 9300)          # smaller still, the other head size
    _case(lib, 12, 20, 5, 128, 1024, 700, 9400)        # larger again: 240 heads, counters beyond the earlier calls'
    _case(lib, 1, 20, 5, 128, 256, 160, 9500)          # short cache: unsplit, the scratch is not touched
    _case(lib, 3, 20, 5, 128, 1536, (1500, 40, 1024), 9600)        # every sequence at its own prefix length


def test_static_scratch_entry_point_in_a_captured_graph():
    """The use the entry point is for: recorded into a HIP graph (after an eager first call on the device) and
    replayed with eager calls and synchronisations in between; every replay must give the eager bits."""
    from ternainfer_amd import _lib
    lib = _lib.load()
    b, h, kv, d, s_max, n = 2, 20, 5, 128, 2048, 1800
    qd, kd, vd, pd, _ = _inputs(b, h, kv, d, s_max, n, 9700)
    scale = float(d) ** -0.5
    eager = torch.zeros((b, h * d), dtype=torch.int16, device="cuda")
    assert lib.ternaspmm_decode_attention_static(_vp(qd), _vp(kd), _vp(vd), _vp(pd), 0, _vp(eager), b, h, kv, d, s_max, scale, None) == 0
    torch.cuda.synchronize()
    out = torch.zeros_like(eager)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    print("[case] decode attention, static scratch, captured", flush=True)
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.ternaspmm_decode_attention_static(_vp(qd), _vp(kd), _vp(vd), _vp(pd), 0, _vp(out), b, h, kv, d, s_max, scale,
                                                       ctypes.c_void_p(side.cuda_stream))
    assert rc == 0
    for replay in range(3):
        out.fill_(-1)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        graph.replay()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(out, eager), f"replay {replay} differs from the eager call"
        _case(lib, 1, 20, 5, 128, 1024, 1000 - replay, 9710 + replay)          # eager work on the same scratch in between
    del graph


def test_static_scratch_entry_point_rejects_what_does_not_fit(capfd):
    from ternainfer_amd import _lib
    lib = _lib.load()
    out = torch.zeros(16, dtype=torch.int16, device="cuda")
    # 13 * 20 = 260 heads > 256: refused before any pointer is touched
    assert lib.ternaspmm_decode_attention_static(None, None, None, None, 0, _vp(out), 13, 20, 5, 128, 1024, 0.1, None) == -1
    assert "exceed" in capfd.readouterr().err
    assert lib.ternaspmm_decode_attention_static(None, None, None, None, 0, _vp(out), 1, 20, 5, 96, 1024, 0.1, None) == -1
    torch.cuda.synchronize()
