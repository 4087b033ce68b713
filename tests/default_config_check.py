"""The library as an unmodified call site gets it -- no environment variable set, the repack cache on -- against the
oracle at the BitNet-2B shapes.  Run by tests/test_gpu_default_config.py in a child process per matrix (the cache
setting is read once per process, and the suite's own process runs with the cache off):

    python -m tests.default_config_check <N> <K> <ws_num>

Every case calls the reference's own symbols on reference-format pointers (kernels/TernaSpMM.cu:25-138, the call
model.py:76-89 makes) at least twice, so that both the first sight of the weight (allocate, repack, reference-format
kernels never run) and the later sights (P2 kernels + fingerprint check) are compared:
  int8 family  bit-exact against the integer oracle, M in {1 (as the padded 8-row call), 8, 16, 256, 2048}, the large
               ones with and without the call site's workspace and on a seeded column sample that straddles every
               weight-scale group boundary;
  bf16 family  within max|err| <= 1e-2 max|ref|, median <= 1 bf16 ULP of the float64 golden, same M;
  one HIP graph captured after the warm-up call, replayed three times with eager calls in between;
  the cache statistics: one copy held while the weight lives, none dropped as stale, none after the clear.
The workspace is exactly as large as the reference's own use of it and is followed by a canary (tests/test_gpu_parity.py).
"""
import ctypes
import os
import sys

import numpy as np
import torch

from oracle import terna_oracle as O
from tests._util import DeviceFormat, make_bf16_activations, make_int8_activations, make_ternary, seed_for, vp
from tests.test_gpu_parity import WS, _check_bf16, run_bf16, run_i8
from ternainfer_amd import _lib


def stats(lib):
    out = (ctypes.c_longlong * 6)()
    lib.ternaspmm_repack_cache_stats(out)
    return list(out)


def main() -> int:
    assert "TERNASPMM_REPACK_CACHE" not in os.environ, "this check is about the library's defaults"
    n, k, ws_num = (int(a) for a in sys.argv[1:4])
    lib = _lib.load()
    assert stats(lib)[0] == 0
    w = make_ternary(n, k, 0.40, seed_for(2, 80 + n % 7))
    fmt = DeviceFormat(w)

    for m in (8, 1, 16):                                          # the first call is the first sight of the weight
        xq, s = make_int8_activations(m, k, seed_for(2, 90 + m))
        mp = max(8, 1 << (m - 1).bit_length())                    # the call site pads rows (model.py:64)
        xq_p = np.concatenate([xq, np.zeros((mp - m, k), np.int8)])
        s_p = np.concatenate([s, O.f32_to_bf16_bits(np.ones(mp - m, np.float32))])
        want = O.spmm_i8(xq, w, s, WS, ws_num, 0)
        for sight in range(2):
            got = run_i8(lib, fmt, xq_p, s_p, WS, ws_num)[:m]
            if not (got == want).all():
                print(f"int8 mismatch M={m} sight={sight}")
                return 1
        x = make_bf16_activations(m, k, seed_for(2, 95 + m))
        scale = np.array([0.7, 1.9, 1.1][:ws_num], np.float32)
        ref = O.spmm_bf16_golden(x, w, scale, ws_num)
        for workspace in (False, True):
            _check_bf16(run_bf16(lib, fmt, x, scale, ws_num, workspace=workspace, split_k=7), ref)
    st = stats(lib)
    assert st[0] == 1 and st[1] == n * k // 4 + 256 + (-(n * k // 4) % 256) and st[2] == 0, st

    rng = np.random.default_rng(seed_for(3, 80 + n % 7))
    edges = [c for b in (2560, 3200, n // 2, n - 1, 0) for c in (b - 1, b, b + 127, b + 128) if 0 <= c < n]
    cols = np.unique(np.concatenate([rng.permutation(n)[:192], np.array(edges)]))
    for m in (256, 2048):
        xq, s = make_int8_activations(m, k, seed_for(3, 85 + m % 97))
        s = s.copy()
        s[m // 3] = 0                                             # the visitor's s == 0 -> coefficient 0 rule
        want = O.spmm_i8(xq, w, s, WS, ws_num, 1, cols=cols)
        first = None
        for workspace in (True, False, True):
            got = run_i8(lib, fmt, xq, s, WS, ws_num, workspace=workspace)
            if not (got[:, cols] == want).all():
                print(f"int8 mismatch M={m} workspace={workspace}")
                return 1
            first = got if first is None else first
            assert (got == first).all(), "split-K and unsplit int8 results must be the same bits"
        x = make_bf16_activations(m, k, seed_for(3, 87 + m % 97), outlier_frac=0.01)
        scale = np.array([1.37, 0.61, 1.9][:ws_num], np.float32)
        gcols = cols[:96]
        grp = O.ws_group_decode(gcols, n, ws_num)
        ref = O.bf16_bits_to_f32(x).astype(np.float64) @ w[gcols].astype(np.float64).T * scale[grp].astype(np.float64)
        for workspace in (True, False):
            _check_bf16(run_bf16(lib, fmt, x, scale, ws_num, workspace=workspace, split_k=7)[:, gcols], ref)

    # one graph captured after the warm-up calls above (the copy exists), replayed with eager work in between
    m = 8
    xq, s = make_int8_activations(m, k, seed_for(2, 99))
    want = O.spmm_i8(xq, w, s, WS, ws_num, 0)
    xd, sd = torch.from_numpy(xq).cuda(), torch.from_numpy(s.view(np.int16)).cuda()
    wsd = torch.from_numpy(WS.view(np.int16)).cuda()
    out = torch.zeros((m, n), dtype=torch.int16, device="cuda")
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    print(f"[case] graph capture on the cached copy N={n} K={k}", flush=True)
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            lib.bitlinear_TernaSpMM(vp(xd), vp(fmt.bm), vp(fmt.off), vp(fmt.med), vp(fmt.vals), vp(out), vp(sd), vp(wsd),
                                    ws_num, m, n, k, 7, None, ctypes.c_void_p(side.cuda_stream))
    for replay in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        if not (out.cpu().numpy().view(np.uint16) == want).all():
            print(f"graph replay {replay} mismatch")
            return 1
        if not (run_i8(lib, fmt, xq, s, WS, ws_num) == want).all():
            print(f"eager call after replay {replay} mismatch")
            return 1
    st = stats(lib)
    assert st[0] == 1 and st[2] == 0 and st[3] == 0, st
    del graph
    lib.ternaspmm_repack_cache_clear()
    assert stats(lib)[:2] == [0, 0]
    print("default configuration check ok")
    return 0


if __name__ == "__main__":
    sys.exit(main())
