"""Run by tests/test_gpu_parity.py::test_repack_cache_behind_reference_entry_points in a child process with
TERNASPMM_REPACK_CACHE=1: the reference-format entry points must give the same results as without the
cache, on first sight (allocate + repack), on later sights (P2 kernels), under graph capture, and after
ternaspmm_repack_cache_clear() when a different weight reuses the same device memory.

With the argument `stale` (a second child process): the weight is rewritten under the same pointers WITHOUT
ternaspmm_repack_cache_clear(); the launch that follows finds a fingerprint that no longer matches, the call after it
drops the copy with a warning and every call from then on serves the new weight (with TERNASPMM_REPACK_CACHE_STRICT=1
that call ends the process with the library's message instead).  The replacement has a SHORTER sign stream than the
original: the check must not sample past its end.

With the argument `limit`: a byte limit that holds two of three weights -- the least recently used copy goes, results
stay right, and a limit below one copy serves every call from the reference format."""
import ctypes
import sys

import numpy as np
import torch

from oracle import terna_oracle as O
from tests._util import DeviceFormat, make_bf16_activations, make_int8_activations, make_ternary, vp
from tests.test_gpu_parity import WS, _check_bf16, run_bf16, run_i8
from ternainfer_amd import _lib


def _stats(lib):
    out = (ctypes.c_longlong * 6)()
    lib.ternaspmm_repack_cache_stats(out)
    return list(out)


def stale() -> int:
    lib = _lib.load()
    # which launch carries the check: the small-M kernel (an extra workgroup, first of the grid), the MFMA-tiled kernel
    # (an extra row of workgroups), or -- with split-K planes in the workspace -- the launch that adds the planes up
    cases = [("small-M kernel", 320, 192, 8, 3, False), ("MFMA-tiled kernel", 320, 192, 300, 4, False),
             ("MFMA-tiled kernel + split-K", 256, 3328, 256, 4, True)]
    for index, (what, n, k, m, kernel, split) in enumerate(cases):
        # the replacement is sparser: its sign stream is shorter than the one the copy's check was set up for
        a, b = DeviceFormat(make_ternary(n, k, 0.30, 980 + index)), DeviceFormat(make_ternary(n, k, 0.70, 990 + index))
        assert b.vals.numel() < a.vals.numel()
        xq, s = make_int8_activations(m, k, 982 + index)
        used = ctypes.c_longlong(0)
        assert lib.ternaspmm_plan_reference_call(1, 0, m, n, k, 7, ctypes.c_void_p(4096), 1, ctypes.byref(used)) == kernel, what
        assert (used.value > 0) == split, (what, used.value)
        for _ in range(2):                           # first sight (copy made), cached sight
            if not (run_i8(lib, a, xq, s, WS, 1) == O.spmm_i8(xq, a.w, s, WS, 1, 0 if m <= 64 else 1)).all():
                print("int8 mismatch before the rewrite", what)
                return 1
        before = _stats(lib)
        a.bm.copy_(b.bm); a.off.copy_(b.off); a.med.copy_(b.med)
        a.vals.zero_(); a.vals[: b.vals.numel()].copy_(b.vals)
        torch.cuda.synchronize()
        print(f"[case] rewritten under the same pointers, no clear: the check rides in the {what}", flush=True)
        run_i8(lib, a, xq, s, WS, 1)                 # this launch reports the stale copy (its result is the old weight's)
        torch.cuda.synchronize()
        want = O.spmm_i8(xq, b.w, s, WS, 1, 0 if m <= 64 else 1)
        for sight in range(3):                       # dropped + rebuilt (first sight again), then cached sights
            if not (run_i8(lib, a, xq, s, WS, 1) == want).all():
                print("the new weight is not served correctly after the stale copy was dropped", what, sight)
                return 1
        st = _stats(lib)
        assert st[2] == before[2] + 1, (what, before, st)
    print("stale copy dropped and rebuilt ok")
    return 0


def limit() -> int:
    lib = _lib.load()
    n, k = 320, 192
    one = n * k // 4 + 256
    assert lib.ternaspmm_repack_cache_limit(2 * one + 100) == -1
    fmts = [DeviceFormat(make_ternary(n, k, 0.40, 990 + j)) for j in range(3)]
    xq, s = make_int8_activations(8, k, 995)
    for order in ([0, 1, 2], [0, 1, 2], [2, 1, 0]):
        for j in order:
            for _ in range(2):
                if not (run_i8(lib, fmts[j], xq, s, WS, 1) == O.spmm_i8(xq, fmts[j].w, s, WS, 1, 0)).all():
                    print("int8 mismatch under the byte limit", order, j)
                    return 1
            st = _stats(lib)
            assert st[0] <= 2 and st[1] <= 2 * one + 100, st
    assert _stats(lib)[3] >= 3, _stats(lib)      # copies were released at the limit
    lib.ternaspmm_repack_cache_clear()
    lib.ternaspmm_repack_cache_limit(one - 1)    # nothing fits: every call is served from the reference format
    for j in range(3):
        if not (run_i8(lib, fmts[j], xq, s, WS, 1) == O.spmm_i8(xq, fmts[j].w, s, WS, 1, 0)).all():
            print("int8 mismatch without room for a copy", j)
            return 1
    assert _stats(lib)[0] == 0
    print("cache limit check ok")
    return 0


def main() -> int:
    if len(sys.argv) > 1 and sys.argv[1] == "stale":
        return stale()
    if len(sys.argv) > 1 and sys.argv[1] == "limit":
        return limit()
    lib = _lib.load()
    co = O.COracle()
    n, k = 320, 192
    weights = [make_ternary(n, k, 0.40, seed) for seed in (950, 951)]
    sources = [DeviceFormat(w) for w in weights]
    fmt = sources[0]                             # its device buffers are reused for the second weight
    shared_vals = torch.zeros(max(f.vals.numel() for f in sources), dtype=fmt.vals.dtype, device="cuda")
    fmt_vals0 = sources[0].vals.clone()
    fmt.vals = shared_vals
    for round_no, w in enumerate(weights):
        src_vals = fmt_vals0 if round_no == 0 else sources[1].vals
        fmt.vals.zero_()
        fmt.vals[: src_vals.numel()].copy_(src_vals)
        if round_no == 1:                        # same device pointers, new contents: the stale-pointer case
            fmt.bm.copy_(sources[1].bm); fmt.off.copy_(sources[1].off); fmt.med.copy_(sources[1].med)
            lib.ternaspmm_repack_cache_clear()
        torch.cuda.synchronize()
        for m in (8, 8, 100, 100):               # first sight, cached sight, both kernel families
            print(f"[case] repack cache weight {round_no} m={m}", flush=True)
            xq, s = make_int8_activations(m, k, 960 + m)
            mode = 0 if m <= 64 else 1
            if not (run_i8(lib, fmt, xq, s, WS, 2) == O.spmm_i8(xq, w, s, WS, 2, mode)).all():
                print("int8 mismatch", round_no, m)
                return 1
            x = make_bf16_activations(m, k, 961 + m)
            scale = np.array([0.7, 1.9], np.float32)
            _check_bf16(run_bf16(lib, fmt, x, scale, 2), co.spmm_bf16(x, w, scale, 2))
    # a weight first seen during capture: served without allocating, replays stay correct
    w = make_ternary(256, 128, 0.40, 970)
    f2 = DeviceFormat(w)
    xq, s = make_int8_activations(8, 128, 971)
    xd = torch.from_numpy(xq).cuda(); sd = torch.from_numpy(s.view(np.int16)).cuda()
    wsd = torch.from_numpy(WS.view(np.int16)).cuda()
    out = torch.zeros((8, 256), dtype=torch.int16, device="cuda")
    work = torch.empty(256 * 128, dtype=torch.int8, device="cuda")
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            lib.bitlinear_TernaSpMM(vp(xd), vp(f2.bm), vp(f2.off), vp(f2.med), vp(f2.vals), vp(out), vp(sd), vp(wsd), 1,
                                    8, 256, 128, 1, vp(work), ctypes.c_void_p(side.cuda_stream))
    for _ in range(2):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        if not (out.cpu().numpy().view(np.uint16) == O.spmm_i8(xq, w, s, WS, 1, 0)).all():
            print("graph replay mismatch")
            return 1
    lib.ternaspmm_repack_cache_clear()
    print("repack cache check ok")
    return 0


if __name__ == "__main__":
    sys.exit(main())
