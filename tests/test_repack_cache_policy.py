"""Host-side logic behind the reference-format entry points, no GPU needed:
  - the repack cache's bookkeeping (csrc/repack_cache.h: identity, least-recently-used release at the byte limit,
    pinned and parked copies, stale copies), compiled with g++ from tests/repack_cache_policy_check.cpp;
  - ternaspmm_plan_reference_call: what a call does with the caller's workspace never exceeds what the reference
    itself writes there (model.py:34-42, tests/test_kernel.cu:331), at every kernel-choice cut."""
import ctypes
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_repack_cache_policy(tmp_path):
    exe = tmp_path / "policy_check"
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", os.path.join(ROOT, "tests", "repack_cache_policy_check.cpp"),
                           "-o", str(exe)])
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and "repack cache policy ok" in r.stdout, r.stdout + r.stderr


SHAPES = [(3840, 2560), (2560, 2560), (13824, 2560), (2560, 6912), (64, 64), (8256, 192), (256, 4160), (128, 6400)]
MS = [1, 8, 16, 32, 33, 48, 64, 65, 96, 128, 129, 192, 193, 256, 257, 512, 2048]


@pytest.mark.parametrize("int8", [1, 0])
@pytest.mark.parametrize("cached", [0, 1])
def test_reference_calls_stay_inside_the_reference_workspace(int8, cached):
    from ternainfer_amd import _lib
    lib = _lib.load()
    aligned, unaligned = ctypes.c_void_p(1 << 20), ctypes.c_void_p((1 << 20) + 8)
    used = ctypes.c_longlong(0)
    kernels_seen, split_seen = set(), 0
    for n, k in SHAPES:
        for m in MS:
            for route in (0, 1, 2):
                for split_k in (1, 2, 7):
                    prefill_path = route == 1 or (route == 0 and m > 64)
                    bound = n * k if prefill_path else 4 * m * n * split_k
                    kern = lib.ternaspmm_plan_reference_call(int8, route, m, n, k, split_k, aligned, cached, ctypes.byref(used))
                    assert 0 <= kern <= 4
                    assert 0 <= used.value <= bound, (int8, cached, n, k, m, route, split_k, kern, used.value, bound)
                    kernels_seen.add(kern)
                    split_seen += used.value > (n * k // 4 if kern == 2 else 0)
                    if kern == 2:                          # the transcode takes the first N*K/4 bytes
                        assert used.value >= n * k // 4 and not cached
                    if cached:
                        assert kern in (3, 4)
                    # no workspace, or one the kernels cannot use: nothing of it is touched
                    for ws in (None, unaligned):
                        kern2 = lib.ternaspmm_plan_reference_call(int8, route, m, n, k, split_k, ws, cached, ctypes.byref(used))
                        assert used.value == 0 and kern2 != 2
                        kernels_seen.add(kern2)
    assert kernels_seen == ({3, 4} if cached else {0, 1, 2})
    assert split_seen > 0                                  # split-K planes do get planned somewhere in the sweep
    assert lib.ternaspmm_plan_reference_call(int8, 0, 8, 100, 64, 7, None, cached, None) == -1


def test_decode_caller_with_few_split_planes_keeps_the_small_kernel_or_fits():
    """tests/test_kernel.cu:331 sizes the workspace as M*N*SPLIT_K*4 bytes: a caller with SPLIT_K = 1 or 2 on a matrix
    of more than 512 bands at M = 33 .. 64 (where the cached path prefers the MFMA-tiled kernel) must not get more
    planes than fit."""
    from ternainfer_amd import _lib
    lib = _lib.load()
    used = ctypes.c_longlong(0)
    for split_k in (1, 2, 3, 7):
        for m in (33, 48, 64):
            kern = lib.ternaspmm_plan_reference_call(1, 0, m, 13824, 2560, split_k, ctypes.c_void_p(4096), 1, ctypes.byref(used))
            assert kern == 4 and used.value <= 4 * m * 13824 * split_k
            assert used.value % (4 * m * 13824) == 0
