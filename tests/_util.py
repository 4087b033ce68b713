"""Shared helpers for the test-suite: seeded synthetic inputs and device plumbing."""
from __future__ import annotations

import ctypes

import numpy as np

from oracle import terna_oracle as O


def seed_for(cfg: int, case: int) -> int:
    return 20260000 + 100 * cfg + case


def make_ternary(n: int, k: int, p0: float, seed: int) -> np.ndarray:
    """iid ternary: P(0)=p0, the rest split evenly between +1 and -1."""
    rng = np.random.default_rng(seed)
    u = rng.random((n, k))
    sgn = rng.random((n, k)) < 0.5
    return np.where(u < p0, 0, np.where(sgn, -1, 1)).astype(np.int8)


def make_row_skewed(n: int, k: int, seed: int) -> np.ndarray:
    """Each output row's zero fraction ~ U[0.2, 0.7]; signs balanced."""
    rng = np.random.default_rng(seed)
    p0 = rng.uniform(0.2, 0.7, size=(n, 1))
    u = rng.random((n, k))
    sgn = rng.random((n, k)) < 0.5
    return np.where(u < p0, 0, np.where(sgn, -1, 1)).astype(np.int8)


def make_bf16_activations(m: int, k: int, seed: int, outlier_frac: float = 0.0) -> np.ndarray:
    """N(0,1) rounded to bf16 storage; optionally a fraction of channels scaled x20."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float32)
    if outlier_frac > 0:
        nch = int(np.ceil(outlier_frac * k))
        ch = rng.permutation(k)[:nch]
        x[:, ch] *= 20.0
    return O.f32_to_bf16_bits(x)


def make_int8_activations(m: int, k: int, seed: int):
    """bf16 N(0,1) activations quantised per row as the call site does -> (int8 [m,k], bf16 s[m])."""
    return O.quant_input(make_bf16_activations(m, k, seed))


def bf16_ulp_distance(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    """Distance in units of bf16 representable steps (sign-magnitude ordered)."""
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


def check_against_fp64(out_bits: np.ndarray, ref: np.ndarray):
    """The tolerance of the bf16 family: max|err| <= 1e-2*max|ref| and median error <= 1 bf16 ULP."""
    got = O.bf16_bits_to_f32(out_bits).astype(np.float64)
    max_ref = np.abs(ref).max()
    max_err = np.abs(got - ref).max()
    ref_bits = O.f32_to_bf16_bits(ref.astype(np.float32))
    ulps = bf16_ulp_distance(out_bits, ref_bits)
    return max_err, max_ref, float(np.median(ulps)), int(ulps.max())


class DeviceFormat:
    """The four format tensors (+ dense ternary W kept on the host) uploaded to the GPU."""

    def __init__(self, w: np.ndarray, device="cuda"):
        import torch
        import ternainfer_amd as T
        self.w = w
        self.n, self.k = w.shape
        vals, off, med, bm = T.compress_weight(torch.from_numpy(w))
        self.host = (vals.numpy(), off.numpy(), med.numpy(), bm.numpy())
        self.vals = vals.to(device) if vals.numel() else torch.zeros(1, dtype=torch.uint32, device=device)[:0]
        self.off = off.to(device)
        self.med = med.to(device)
        self.bm = bm.to(device)

    @property
    def n_sign_words(self) -> int:
        return int(self.host[0].size)


def vp(t):
    return ctypes.c_void_p(t.data_ptr())
