#!/usr/bin/env python3
"""Benchmark of the TernaSpMM path on one MI355X.

A step is one decode pass over the BitNet-b1.58-2B ternary layer set -- QKV 2560->3840,
O 2560->2560, gate+up 2560->13824, down 6912->2560 -- for `--layers` layers (default 30, the
model's depth) at M = `--m` activation rows (default 8), bf16 activations, fp32 accumulate, one
fp32 scale per matrix.  Every layer has its own copy of the compressed weights, so one step
streams ~417 MB of distinct weight bytes: more than the 256 MB last-level cache, i.e. the
weights come from HBM on every step ("cold stream").  The step is captured once in a HIP graph
(as the reference's generate.py does for its forward) and replayed.

Prints ONE JSON line.  `value` is algorithmic GB/s: bytes of the reference-format tensors
(bitmaps, sign words, both offset arrays), activations in, scales, bf16 out -- never the
dense matrix -- divided by the measured time.  `roofline` prices the same bytes against the
8 TB/s HBM peak; `cpu_baseline` times decode-to-dense + torch.matmul on the host cores for one
layer of the same workload and doubles as the correctness gate of the run.

The default run (`--workload decode`) also measures, in the same process and into the same line,
the other figures of the path: the literal single-matrix configuration (`config1`),
the layer set at M = 1 and 16, the same launches without the dependence between them (`launches_overlapped`,
evidence only), the unmodified call site (`drop_in_reference_format`), the prefill
shapes at M = 2048 for both activation types (`prefill_m2048`), the 2B-shaped model's decode
tokens/s at batch 1 and 8 and, for one sequence, far into a 2048-slot context (`model_decode`) and what the machine gives (`calibration`: cost of a
graph kernel node, read and copy rate, cost of a device-wide synchronisation).  `--no-extras`
leaves those out.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
BF16_MFMA_PEAK_TFLOPS = 2500.0
INT8_MFMA_PEAK_TOPS = 5000.0
LAYER_SET = [("wqkv", 3840, 2560), ("wo", 2560, 2560), ("w13", 13824, 2560), ("w2", 2560, 6912)]   # (name, N, K)
METRIC = "TernaSpMM GB/s + %HBM roofline (M=8,K=N=2560); 2B-shape decode tok/s"

# HBM bytes per launch of the small-M P2 kernel on the default workload (M=8, average over the four matrices):
# a counter measurement, not part of this run -- two rocprofv3 --pmc runs of this file (FETCH_SIZE, WRITE_SIZE),
# scaled by what the same counters read for a 256 MiB copy.  Quoted with its source; null for any other workload.
TRAFFIC = {"bytes_per_launch": (19046.0 + 356.0) * 1024 / 4,
           "source": "profiles/decode_chunk_kernels_hbm_traffic.md (two rocprofv3 --pmc runs, FETCH_SIZE x 2.0 and WRITE_SIZE x 1.0 by the copy probe)",
           "measured_at": "the tree of the commit 'O projection of the chained step in the wide-load form ...' "
                          "(csrc/decode_chunk_kernel.h and launch_decode_packed.hip as of 'Small-M kernel with four band-tiles per weight load ...')"}


def vp(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def make_ternary(n, k, p0, seed):
    """iid ternary from 16-bit draws: zero iff draw < p0 * 65536 (P(0) = p0 to 1e-5), sign = bit 0,
    which is balanced and independent of the zero test."""
    rng = np.random.default_rng(seed)
    b = rng.integers(0, 65536, size=(n, k), dtype=np.uint16)
    nz = (b >= np.uint16(int(p0 * 65536))).astype(np.int8)
    return nz * (1 - 2 * (b & 1).astype(np.int8))


def f32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def make_row_skewed(n, k, seed):
    """Each output row's zero fraction drawn U[0.2, 0.7]; signs balanced (configs[3])."""
    rng = np.random.default_rng(seed)
    p0 = rng.uniform(0.2, 0.7, size=(n, 1))
    nz = (rng.random((n, k)) >= p0).astype(np.int8)
    return nz * (1 - 2 * rng.integers(0, 2, size=(n, k), dtype=np.int8))


class Matrix:
    """One ternary matrix: host copy, `copies` device copies of the format (reference layout and P2),
    and per activation-row count M a bf16 activation block and an output."""

    def __init__(self, name, n, k, m, copies, seed, torch, T, w=None, p0=0.40):
        self.torch = torch
        self.name, self.n, self.k, self.m = name, n, k, m
        self.w = make_ternary(n, k, p0, seed) if w is None else w
        vals, off, med, bm = T.compress_weight(torch.from_numpy(self.w))
        self.host_format = (vals.numpy(), off.numpy(), med.numpy(), bm.numpy())
        self.n_sign_words = int(vals.numel())
        base = [t.cuda() for t in (vals, off, med, bm)]
        self.dev = [base] + [[t.clone() for t in base] for _ in range(copies - 1)]
        lib = T._lib.load()
        self.packed = []                     # load-time repack (P2 layout), one buffer per weight copy
        for vals_d, off_d, med_d, bm_d in self.dev:
            buf = torch.empty(lib.ternaspmm_packed_bytes(n, k) // 4, dtype=torch.int32, device="cuda")
            lib.ternaspmm_repack(vp(bm_d), vp(off_d), vp(med_d), vp(vals_d), vp(buf), n, k, None)
            self.packed.append(buf)
        torch.cuda.synchronize()
        self.seed = seed
        rng = np.random.default_rng(seed + 1)
        self.x_bits = f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
        self.scale_host = rng.uniform(0.5, 2.0, 1).astype(np.float32)
        self.scale = torch.from_numpy(self.scale_host).cuda()
        self.acts = {m: (torch.from_numpy(self.x_bits.view(np.int16)).cuda(), torch.zeros((m, n), dtype=torch.int16, device="cuda"))}
        self.x, self.out = self.acts[m]

    def bytes_at(self, m):
        """Reference-format bytes one call at M = m has to move."""
        n, k = self.n, self.k
        return (8 * (n * k // 64) + 4 * self.n_sign_words + 4 * (n * k // 4096 + 1) + 2 * (3 * n * k // 4096)
                + 2 * m * k + 4 + 2 * m * n)

    @property
    def alg_bytes(self):
        return self.bytes_at(self.m)

    def act(self, m):
        if m not in self.acts:
            rng = np.random.default_rng(self.seed + 100 + m)
            x = f32_to_bf16_bits(rng.standard_normal((m, self.k)).astype(np.float32))
            self.acts[m] = (self.torch.from_numpy(x.view(np.int16)).cuda(),
                            self.torch.zeros((m, self.n), dtype=self.torch.int16, device="cuda"))
        return self.acts[m]

    def launch(self, lib, copy, stream, layout="packed", m=None):
        m = self.m if m is None else m
        x, out = self.act(m)
        if layout == "packed":
            lib.bitlinear_TernaSpMM_bf16_packed(vp(x), vp(self.packed[copy]), vp(out), vp(self.scale), 1, m, self.n, self.k, 0, stream)
        else:
            vals, off, med, bm = self.dev[copy]
            lib.bitlinear_TernaSpMM_bf16(vp(x), vp(bm), vp(off), vp(med), vp(vals), vp(out), vp(self.scale),
                                         1, m, self.n, self.k, 1, None, stream)


def golden_gate(mats, what):
    """The correctness gate of a timed leg, on the outputs its launches left: every matrix against the float64
    evaluation of X (bf16) x W^T (the host's ternary matrix) x scale, max |err| <= 1e-2 max |ref| and a median error of
    at most one bf16 step.  numpy only.  Returns max err / max |ref| per matrix."""
    ratios = {}
    for mat in mats:
        x = (mat.x_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        golden = x @ mat.w.astype(np.float64).T * float(mat.scale_host[0])
        bits = mat.out.cpu().numpy().view(np.uint16)
        got = (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        max_ref, max_err = np.abs(golden).max(), np.abs(got - golden).max()
        assert max_err <= 1e-2 * max_ref, f"{what}, {mat.name}: max_err {max_err} vs max_ref {max_ref}"
        want = f32_to_bf16_bits(golden.astype(np.float32)).astype(np.int32)
        key = lambda u: np.where(u & 0x8000, -(u & 0x7FFF), u & 0x7FFF)
        assert np.median(np.abs(key(bits.astype(np.int32)) - key(want))) <= 1, f"{what}, {mat.name}: median error above one bf16 step"
        ratios[mat.name] = float(max_err / max_ref)
    return ratios


def time_graph(torch, graph, replays, warmup, sustain_ms=0.0):
    """ms per replay over `replays` replays after `warmup` untimed ones.  sustain_ms > 0: the untimed replays go on until
    that much wall time has passed -- a chip that idled while the host built data needs tens of milliseconds of matrix
    load before it runs in its sustained state (measured: the M = 2048 step reads 270 us in the first 15 ms after an idle
    phase and 245 us from then on, whatever is measured; the small-M launches do not move)."""
    for _ in range(warmup):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while sustain_ms > 0.0 and (time.perf_counter() - t0) * 1e3 < sustain_ms:
        for _ in range(8):
            graph.replay()
        torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(replays):
        graph.replay()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / replays       # ms per replay


def capture(torch, fn):
    """Capture fn(stream_handle) into a graph on a side stream (events are recorded on the
    stream the replays are issued to, the current one)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            fn(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.current_stream().wait_stream(side)
    return g


def cpu_baseline(mats, torch):
    """Decode the compressed format to dense on the host (C oracle, one thread), then
    torch.matmul(X.float(), W.T) * scale on all host cores; one layer set per repetition, repeated for about ten
    seconds of CPU work (at least five times), median.
    Also the correctness gate: the GPU outputs of layer copy 0 must match this golden."""
    from oracle import terna_oracle as O
    orc = O.COracle()
    # the GPU box grants a share of its host cores and exports it as OMP_NUM_THREADS
    cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    t_decode, t_matmul, alg = [], [], 0
    parity = {}
    for mat in mats:
        alg += mat.alg_bytes
    t_begin = time.perf_counter()
    rep = -1
    while rep < 4 or (time.perf_counter() - t_begin < 10.0 and rep < 199):
        rep += 1
        td = tm = 0.0
        for mat in mats:
            t0 = time.perf_counter()
            w = orc.decode(*mat.host_format, mat.n, mat.k)
            t1 = time.perf_counter()
            xf = torch.from_numpy(O.bf16_bits_to_f32(mat.x_bits))
            wf = torch.from_numpy(w).float()
            ref = torch.matmul(xf, wf.t()) * float(mat.scale_host[0])
            t2 = time.perf_counter()
            td += t1 - t0
            tm += t2 - t1
            if rep == 0:
                assert (w == mat.w).all(), f"{mat.name}: decode(encode(W)) != W"
                golden = O.spmm_bf16_golden(mat.x_bits, w, mat.scale_host, 1)
                got = O.bf16_bits_to_f32(mat.out.cpu().numpy().view(np.uint16)).astype(np.float64)
                max_ref = np.abs(golden).max()
                max_err = np.abs(got - golden).max()
                assert max_err <= 1e-2 * max_ref, f"{mat.name}: max_err {max_err} vs max_ref {max_ref}"
                assert np.abs(ref.double().numpy() - golden).max() <= 1e-3 * max_ref
                parity[mat.name] = float(max_err / max_ref)
        t_decode.append(td)
        t_matmul.append(tm)
    total = float(np.median(np.array(t_decode) + np.array(t_matmul)))
    return {
        "value": alg / total / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
        "sample": (f"one layer set (4 matrices, M={mats[0].m}), median of {len(t_decode)} repetitions "
                   f"({time.perf_counter() - t_begin:.1f} s of CPU work): C-oracle decode to dense on 1 thread "
                   f"({float(np.median(t_decode)) * 1e3:.1f} ms) + torch.matmul fp32 on {cores} threads "
                   f"({float(np.median(t_matmul)) * 1e3:.1f} ms)"),
        "decode_ms": float(np.median(t_decode)) * 1e3, "matmul_ms": float(np.median(t_matmul)) * 1e3,
        "parity_max_err_over_max_ref": parity,
    }


# ------------------------------------------------------------------------------------------------ model (configs[4])
def measure_model(torch, batch, act="int8", prefetch=True, gen_tokens=256, check_tokens=8, model=None, prompt_tokens=128, chain=True):
    """2B-shaped random-init model, prompt of `prompt_tokens` (128) uniform random ids, greedy decode of `gen_tokens`
    tokens; tokens/s = generated tokens / decode-phase time (as the reference's stats.py:19-27).
    Self-check of the run: the captured decode graph must produce the tokens of eager execution
    for the first `check_tokens` tokens.  Returns (figures, model)."""
    from ternainfer_amd.model import ModelArgs, Transformer, greedy_decode
    margs = ModelArgs()
    t0 = time.perf_counter()
    if model is None:
        model = Transformer(margs, seed=20260500, act=act)
    model.chain = chain
    if os.environ.get("TERNA_BENCH_CHAIN_ROWS"):           # measurement aids
        model.chain_rows = int(os.environ["TERNA_BENCH_CHAIN_ROWS"])
    if os.environ.get("TERNA_BENCH_SPLIT_ROWS"):
        model.split_rows = int(os.environ["TERNA_BENCH_SPLIT_ROWS"])
    if os.environ.get("TERNA_BENCH_ATTN_SPLITS"):
        model.attention_splits = int(os.environ["TERNA_BENCH_ATTN_SPLITS"])
    if os.environ.get("TERNA_BENCH_SPLIT_MERGE_QUANT"):
        model.split_merge_quant = os.environ["TERNA_BENCH_SPLIT_MERGE_QUANT"] != "0"
    if os.environ.get("TERNA_BENCH_STEP_INPUTS"):
        model.step_inputs = os.environ["TERNA_BENCH_STEP_INPUTS"] != "0"
    if os.environ.get("TERNA_BENCH_DEFER_ABOVE"):
        model.defer_above = int(os.environ["TERNA_BENCH_DEFER_ABOVE"])
    if os.environ.get("TERNA_BENCH_ATTENTION_STATS"):
        for blk in model.layers:
            blk.attention_stats = os.environ["TERNA_BENCH_ATTENTION_STATS"] != "0"
    if os.environ.get("TERNA_BENCH_ATTENTION_STATS_CHAIN"):
        for blk in model.layers:
            blk.attention_stats_chain = os.environ["TERNA_BENCH_ATTENTION_STATS_CHAIN"] != "0"
    if os.environ.get("TERNA_BENCH_O_NORM_ROWS"):
        for blk in model.layers:
            blk.o_norm_rows = int(os.environ["TERNA_BENCH_O_NORM_ROWS"])
    if os.environ.get("TERNA_BENCH_CHAIN_MERGE_QUANT"):
        for blk in model.layers:
            blk.merge_quant = os.environ["TERNA_BENCH_CHAIN_MERGE_QUANT"] != "0"
    if os.environ.get("TERNA_BENCH_CHAIN_DOWN_ROWS"):
        for blk in model.layers:
            blk.chain_down_rows = int(os.environ["TERNA_BENCH_CHAIN_DOWN_ROWS"])
    model.enable_prefetch(False)
    if prefetch and batch <= 2:     # weights of the following launches, pulled through the caches during the attention launch
        model.enable_prefetch(True, ("wo", "w13", "w2", "next_wqkv", "norms"))
    torch.cuda.synchronize()
    build_s = time.perf_counter() - t0
    gen = torch.Generator(device="cuda").manual_seed(20260501)
    prompt = torch.randint(0, margs.vocab_size, (batch, prompt_tokens), generator=gen, device="cuda")
    warm, _, _ = greedy_decode(model, prompt, check_tokens)                     # warm-up (code objects, allocator)
    eager, _, _ = greedy_decode(model, prompt, check_tokens, use_graph=False)
    graph_equals_eager = bool(torch.equal(warm, eager))
    assert graph_equals_eager, "decode graph and eager execution disagree"
    toks, prefill_s, decode_s = greedy_decode(model, prompt, gen_tokens)
    assert torch.equal(toks[:, :check_tokens], eager)
    return {"batch": batch, "tokens_per_s": batch * gen_tokens / decode_s, "ms_per_step": decode_s * 1e3 / gen_tokens,
            "prefill_tokens_per_s": batch * prompt_tokens / prefill_s, "prefill_ms": prefill_s * 1e3, "decode_s": decode_s,
            "prompt_tokens": prompt_tokens,
            "generated_tokens": gen_tokens, "graph_equals_eager_first_tokens": check_tokens,
            "first_tokens": toks[0, :8].tolist(), "model_build_s": build_s}, model


def run_model(args, torch):
    act = args.act or "int8"
    gen = 256 if args.prompt_tokens <= 128 else 128
    fig, _ = measure_model(torch, args.batch, act, not args.no_prefetch, gen_tokens=gen, prompt_tokens=args.prompt_tokens,
                           chain=not args.no_chain)
    return {
        "metric": "2B-shape decode tok/s", "value": fig["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": gen, "warmup": 8,
        "ms_per_step": fig["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": act, "data": "synthetic",
        "config": {"workload": f"configs[4]: BitNet-b1.58-2B-shaped random-init decoder (30 layers, hidden 2560, 20/5 heads, "
                               f"FFN 6912, vocab 128256), batch {args.batch}, {args.prompt_tokens}-token prompt, {gen} greedy tokens, "
                               f"{act} activations into the ternary linears, weights in P2 layout, one HIP graph per "
                               "decode step; norms, gate, activation quantisation, RoPE, cache write, single-token "
                               "attention, the multi-token attention of the prompt pass, the bf16 LM head and greedy "
                               "sampling are library kernels; the prompt pass is one HIP graph too"
                               + ("; one sequence: the attention is split over several workgroups per head and the O "
                                  "projection's prologue merges the partial results" if args.batch == 1 else
                                  ("" if args.no_prefetch or args.batch > 2 else "; the idle CUs of the attention launch "
                                                                                 "prefetch the weights of the launches that follow"))
                               + ("" if args.no_chain or args.batch > 8 else
                                  "; the linears are chained through producer-side norm statistics"
                                  + (" (consumed inside the next linear)" if args.batch <= 4 else
                                     " (consumed by an element-wise quantise launch in front of the next linear)")),
                   "batch": args.batch, "act": act},
        **{k: fig[k] for k in ("prefill_tokens_per_s", "prefill_ms", "decode_s", "model_build_s", "first_tokens",
                               "graph_equals_eager_first_tokens")}}


# ------------------------------------------------------------------------------------------------ sweep (configs[3])
def run_sweep(args, torch, T, lib):
    """configs[3]: sparsity / structure sweep at M = 16 on K = N = 2560 and on K = 6912, N = 2560 -- global zero
    fraction 0.20 / 0.33 / 0.45 / 0.60 and a row-skewed matrix -- on both weight layouts.  The reference format's
    size, and with it the work of the kernels that read it, follows the number of nonzeros; the 2-bit layout and
    its kernels do not.  A step is one pass over the ten matrices (cold: --layers copies of each, rotated)."""
    m = args.m if args.m != 8 else 16
    copies = min(args.layers, 24)
    from oracle import terna_oracle as O
    cases, mats = [], []
    for n, k in [(2560, 2560), (2560, 6912)]:
        for kind in ["p20", "p33", "p45", "p60", "skewed"]:
            seed = 20260400 + len(cases)
            w = make_row_skewed(n, k, seed) if kind == "skewed" else make_ternary(n, k, int(kind[1:]) / 100.0, seed)
            cases.append((f"{kind}_{k}x{n}", float((w == 0).mean())))
            mats.append(Matrix(cases[-1][0], n, k, m, copies, seed, torch, T, w=w))
    detail, total_bytes, total_us = {}, 0, {"packed": 0.0, "reference": 0.0}
    for (name, zero_frac), mt in zip(cases, mats):
        entry = {"zero_fraction": zero_frac, "alg_bytes": mt.alg_bytes}
        for layout in ("packed", "reference"):
            g = capture(torch, lambda s, mt=mt, layout=layout: [mt.launch(lib, c, s, layout) for c in range(copies)])
            us = time_graph(torch, g, max(args.steps // 2, 5), args.warmup) * 1e3 / copies
            entry[f"{layout}_us"] = us
            entry[f"{layout}_GBps"] = mt.alg_bytes / us / 1e3
            total_us[layout] += us
            # correctness gate of the run: the last launch's output against the fp64 golden
            gold = O.spmm_bf16_golden(mt.x_bits, mt.w, mt.scale_host, 1)
            got = O.bf16_bits_to_f32(mt.out.cpu().numpy().view(np.uint16)).astype(np.float64)
            assert np.abs(got - gold).max() <= 1e-2 * np.abs(gold).max(), (name, layout)
        detail[name] = entry
        total_bytes += mt.alg_bytes
    gbps = total_bytes / total_us[args.layout] / 1e3
    return {
        "metric": METRIC, "value": gbps, "unit": "GB/s",
        "n_gpus": 1, "steps": max(args.steps // 2, 5), "warmup": args.warmup, "ms_per_step": total_us[args.layout] * 1e-3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"configs[3]: sparsity / structure sweep, M={m}, K=N=2560 and K=6912 N=2560, zero fraction "
                               f"0.20 / 0.33 / 0.45 / 0.60 and row-skewed U[0.2, 0.7]; {copies} weight copies per matrix, "
                               f"value = the ten matrices on the {args.layout} layout",
                   "m": m, "layout": args.layout},
        "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS,
                     "traffic": None},
        "per_case": detail}


# ------------------------------------------------------------------------------------------------ prefill (configs[2])
class PrefillSet:
    """The four BitNet-2B matrices with activations at the given row counts: bf16 with 1% of the channels
    scaled x20, and the same activations quantised per row to int8 (the reference's own prefill input)."""

    def __init__(self, torch, T, m_values, acts=("bf16", "int8")):
        self.torch = torch
        rng = np.random.default_rng(20260300)
        self.mats = []
        for j, (name, n, k) in enumerate(LAYER_SET):
            mt = Matrix(name, n, k, 8, 1, 20260300 + 10 * j, torch, T)
            xs = {}
            for m in sorted(set(m_values)):
                xf = rng.standard_normal((m, k)).astype(np.float32)
                ch = rng.permutation(k)[: int(np.ceil(0.01 * k))]
                xf[:, ch] *= 20.0
                if "bf16" in acts:
                    xs[("bf16", m)] = (torch.from_numpy(f32_to_bf16_bits(xf).view(np.int16)).cuda(),
                                       torch.zeros((m, n), dtype=torch.int16, device="cuda"))
                if "int8" in acts:     # per-row absmax quantisation, as the reference's quant_input (model.py:120-123)
                    sc = 127.0 / np.maximum(np.abs(xf).max(axis=1, keepdims=True), 1e-5)
                    xq = np.clip(np.rint(xf * sc), -128, 127).astype(np.int8)
                    xs[("int8", m)] = (torch.from_numpy(xq).cuda(), torch.zeros((m, n), dtype=torch.int16, device="cuda"),
                                       torch.from_numpy(f32_to_bf16_bits(sc.astype(np.float32).ravel()).view(np.int16)).cuda())
            mt.ws = torch.from_numpy(f32_to_bf16_bits(mt.scale_host).view(np.int16)).cuda()
            self.mats.append((mt, xs))
        self.work = torch.empty(13824 * 2560, dtype=torch.int8, device="cuda")      # the reference's global workspace

    def launch(self, lib, mt, xs, act, m, s, layout="packed", route=0):
        if act == "int8":
            x, out, srow = xs[("int8", m)]
            if layout == "packed":
                lib.bitlinear_TernaSpMM_packed_ws(vp(x), vp(mt.packed[0]), vp(out), vp(srow), vp(mt.ws), 1, m, mt.n, mt.k, route,
                                                  vp(self.work), self.work.numel(), s)
            else:
                vals, off, med, bm = mt.dev[0]
                lib.bitlinear_TernaSpMM(vp(x), vp(bm), vp(off), vp(med), vp(vals), vp(out), vp(srow), vp(mt.ws), 1, m, mt.n, mt.k,
                                        7, vp(self.work), s)
            return
        x, out = xs[("bf16", m)]
        if layout == "packed":
            lib.bitlinear_TernaSpMM_bf16_packed_ws(vp(x), vp(mt.packed[0]), vp(out), vp(mt.scale), 1, m, mt.n, mt.k, route,
                                                   vp(self.work), self.work.numel(), s)
        else:                      # reference-format pointers + workspace: transcode per call, then the P2 kernel
            vals, off, med, bm = mt.dev[0]
            lib.bitlinear_TernaSpMM_bf16(vp(x), vp(bm), vp(off), vp(med), vp(vals), vp(out), vp(mt.scale),
                                         1, m, mt.n, mt.k, 1, vp(self.work), s)

    def dense_us(self, act, m, n, k, reps=10):
        """Vendor dense GEMM of the same shape on expanded weights (a yardstick, not part of the product)."""
        torch = self.torch
        if act == "bf16":
            a = torch.randn(m, k, device="cuda", dtype=torch.bfloat16)
            b = torch.randn(n, k, device="cuda", dtype=torch.bfloat16).t()
            f = lambda: torch.matmul(a, b)
        else:
            a = torch.randint(-127, 128, (m, k), device="cuda", dtype=torch.int8)
            b = torch.randint(-1, 2, (n, k), device="cuda", dtype=torch.int8).t()
            f = lambda: torch._int_mm(a, b)
        try:
            for _ in range(3):
                f()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                f()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3 / reps
        except Exception:                                   # no such vendor kernel in this build
            return None

    def shape_us(self, lib, mt, xs, act, m, layout="packed", route=0, reps=10, replays=5, warmup=2):
        torch = self.torch
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        self.launch(lib, mt, xs, act, m, stream, layout, route)
        torch.cuda.synchronize()
        g = capture(torch, lambda s: [self.launch(lib, mt, xs, act, m, s, layout, route) for _ in range(reps)])
        return time_graph(torch, g, replays, warmup) * 1e3 / reps

    def step(self, lib, act, m, steps, warmup, layout="packed"):
        """One pass over the four matrices at M = m, graph-replayed: (ms per step, flops per step)."""
        torch = self.torch
        graph = capture(torch, lambda s: [self.launch(lib, mt, xs, act, m, s, layout) for mt, xs in self.mats])
        ms = time_graph(torch, graph, steps, warmup, sustain_ms=60.0)
        return ms, sum(2.0 * m * mt.n * mt.k for mt, _ in self.mats)

    def dense_step(self, act, m, steps, warmup):
        """The vendor's dense GEMM on the same four shapes in the SAME protocol: one graph of the four calls (operands
        and outputs allocated beforehand), replayed `steps` times after `warmup`.  ms per step, or None."""
        torch = self.torch
        try:
            ops = []
            for mt, _ in self.mats:
                if act == "bf16":
                    a = torch.randn(m, mt.k, device="cuda", dtype=torch.bfloat16)
                    b = torch.randn(mt.n, mt.k, device="cuda", dtype=torch.bfloat16).t()
                    o = torch.empty(m, mt.n, device="cuda", dtype=torch.bfloat16)
                    ops.append((torch.matmul, a, b, o))
                else:
                    a = torch.randint(-127, 128, (m, mt.k), device="cuda", dtype=torch.int8)
                    b = torch.randint(-1, 2, (mt.n, mt.k), device="cuda", dtype=torch.int8).t()
                    o = torch.empty(m, mt.n, device="cuda", dtype=torch.int32)
                    ops.append((torch._int_mm, a, b, o))
            run = lambda: [f(a, b, out=o) for f, a, b, o in ops]
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                run()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                run()
            return time_graph(torch, g, steps, warmup, sustain_ms=60.0)
        except Exception:                                   # no such vendor kernel in this build
            return None


def prefill_figures(ps, lib, act, m, steps, warmup, per_shape=True, layout="packed"):
    peak = BF16_MFMA_PEAK_TFLOPS if act == "bf16" else INT8_MFMA_PEAK_TOPS
    ms, flops = ps.step(lib, act, m, steps, warmup, layout)
    rate = flops / (ms * 1e-3) / 1e12
    out = {"act": act, "m": m, "ms_per_step": ms, "rate": rate, "unit": "TFLOP/s" if act == "bf16" else "TOP/s",
           "peak": peak, "frac": rate / peak}
    if per_shape:
        shapes, dense_total, own_total = {}, 0.0, 0.0
        for mt, xs in ps.mats:
            us = ps.shape_us(lib, mt, xs, act, m, layout, replays=10, warmup=3)           # 100 timed launches per shape
            d_us = ps.dense_us(act, m, mt.n, mt.k, reps=30)
            tf = 2.0 * m * mt.n * mt.k / us / 1e6
            shapes[f"{mt.name}_{mt.k}x{mt.n}"] = {"us": us, "rate": tf, "frac": tf / peak, "vendor_dense_gemm_us": d_us}
            dense_total = None if (d_us is None or dense_total is None) else dense_total + d_us
            own_total += us
        out["per_shape"] = shapes
        # the step (a graph of the four launches, one after the other) and the sum of the four shapes timed alone,
        # side by side: the clock under matrix load moves the former more than the latter
        out["per_shape_sum"] = {"ms": own_total * 1e-3, "rate": flops / (own_total * 1e-6) / 1e12,
                                "frac": flops / (own_total * 1e-6) / 1e12 / peak}
        d_ms = ps.dense_step(act, m, steps, warmup)
        out["vendor_dense_gemm"] = None if (not dense_total and d_ms is None) else {
            "what": "torch.matmul (bf16) / torch._int_mm (int8) on already expanded weights, same four shapes: "
                    "ms_per_step = one graph of the four calls, timed exactly as this kernel's step; per_shape_sum_ms = "
                    "the four shapes timed alone (eager, 30 calls each)",
            "ms_per_step": d_ms, "rate": None if d_ms is None else flops / (d_ms * 1e-3) / 1e12,
            "per_shape_sum_ms": None if not dense_total else dense_total * 1e-3,
            "per_shape_sum_rate": None if not dense_total else flops / (dense_total * 1e-6) / 1e12}
    return out


def run_prefill(args, torch, T, lib):
    """configs[2]: the four BitNet-2B matrices at M in {256, 512, 2048}, bf16 activations with 1% of
    the channels scaled x20 (--act int8: the same activations quantised per row to int8, the
    reference's own prefill input).  A step is one pass over the four matrices at M = --m (default
    2048 when --workload prefill is given without --m).  Next to every shape the vendor's dense GEMM
    (torch.matmul / torch._int_mm on already expanded weights) is timed as a yardstick."""
    m_main = args.m if args.m >= 64 else 2048
    act = args.act or "bf16"
    ms_all = sorted({256, 512, 2048, m_main})
    ps = PrefillSet(torch, T, [m_main] if args.no_per_shape else ms_all, acts=(act,))
    fig = prefill_figures(ps, lib, act, m_main, args.steps, args.warmup, per_shape=False, layout=args.layout)
    per_shape, dense_main = {}, None
    if not args.no_per_shape:
        peak = fig["peak"]
        dense_main = 0.0
        for mt, xs in ps.mats:
            for m in ms_all:
                us = ps.shape_us(lib, mt, xs, act, m, args.layout)
                d_us = ps.dense_us(act, m, mt.n, mt.k)
                tf = 2.0 * m * mt.n * mt.k / us / 1e6
                per_shape[f"{mt.name}_{mt.k}x{mt.n}_M{m}"] = {"us": us, "tflops": tf, "frac": tf / peak, "vendor_dense_gemm_us": d_us}
                if m == m_main:
                    dense_main = None if (d_us is None or dense_main is None) else dense_main + d_us
    flops = sum(2.0 * m_main * mt.n * mt.k for mt, _ in ps.mats)
    unit = fig["unit"]
    return {
        "metric": "TernaSpMM prefill TFLOP/s + %bf16 MFMA peak (M=2048, BitNet-2B layer set)" if act == "bf16"
                  else "TernaSpMM prefill TOP/s, int8 activations (M=2048, BitNet-2B layer set)",
        "value": fig["rate"], "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": fig["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if act == "bf16" else "int8", "data": "synthetic",
        "config": {"workload": f"configs[2]: four BitNet-b1.58-2B matrices at M={m_main}, P(0)=0.40, {act} activations "
                               "with 1% outlier channels (x20), HIP-graph replay; weight layout: "
                               + ("P2, repacked once at load time" if args.layout == "packed"
                                  else "reference format, transcoded into the workspace on every call"),
                   "m": m_main, "layout": args.layout},
        "roofline": {"bound": "mfma", "achieved": fig["rate"], "peak": fig["peak"], "unit": unit, "frac": fig["frac"], "traffic": None,
                     "kernel": f"terna_prefill_packed_dma_kernel<{act}>", "algorithmic_flops_per_step": flops},
        "vendor_dense_gemm": None if not dense_main else {
            "what": "torch.matmul (bf16) / torch._int_mm (int8) on already expanded weights, same four shapes, eager",
            "ms_per_step": dense_main * 1e-3, "rate": flops / (dense_main * 1e-6) / 1e12},
        "per_shape": per_shape}


# ------------------------------------------------------------------------------------------------ mid-M policy
def run_midm(args, torch, T, lib):
    """Both kernel families (route 2 = small-M dot-product kernel, route 1 = MFMA-tiled kernel) on the four 2B
    matrices at the batch sizes between decode and prefill, P2 layout, hot (one weight copy: the choice of
    kernel is about the compute side).  The library's own choice (route 0) is timed beside them."""
    m_values = [16, 24, 32, 48, 64, 96, 128, 192, 256]
    act = args.act or "bf16"
    ps = PrefillSet(torch, T, m_values, acts=(act,))
    table = {}
    for mt, xs in ps.mats:
        for m in m_values:
            row = {}
            routes = (("small_m_kernel_us", 2), ("mfma_kernel_us", 1), ("library_choice_us", 0)) if act == "bf16" else \
                     (("small_m_kernel_us", 4), ("mfma_kernel_us", 8), ("library_choice_us", 0))     # int8: +4 / +8 pick the kernel
            for label, route in routes:
                row[label] = ps.shape_us(lib, mt, xs, act, m, "packed", route)
            row["best"] = "small_m" if row["small_m_kernel_us"] <= row["mfma_kernel_us"] else "mfma"
            table[f"{mt.name}_{mt.k}x{mt.n}_M{m}"] = row
    worst = max(r["library_choice_us"] / min(r["small_m_kernel_us"], r["mfma_kernel_us"]) for r in table.values())
    return {"metric": "TernaSpMM mid-M kernel choice (us per launch)", "value": worst, "unit": "library choice / best, worst case",
            "n_gpus": 1, "steps": 5, "warmup": 2, "ms_per_step": None, "higher_is_better": False, "scaling": "weak",
            "vs_baseline": None, "dtype": act, "data": "synthetic",
            "config": {"workload": f"four BitNet-b1.58-2B matrices at M in {m_values}, {act} activations, P2 layout, hot"},
            "per_shape": table}


# ------------------------------------------------------------------------------------------------ calibration
def calibration(torch, lib):
    """What the machine gives, measured by the library's own probe kernels in this run."""
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    nodes = 1000
    g = capture(torch, lambda s: [lib.ternaspmm_probe_empty(s) for _ in range(nodes)])
    out["graph_kernel_node_us"] = time_graph(torch, g, 5, 2) * 1e3 / nodes
    nbytes = 1 << 30
    a = torch.empty(nbytes, dtype=torch.int8, device="cuda").fill_(1)
    b = torch.empty(nbytes, dtype=torch.int8, device="cuda")
    for name, fn, moved in (("read_GBps", lambda: lib.ternaspmm_probe_read(vp(a), nbytes, None, stream), nbytes),
                            ("copy_GBps", lambda: lib.ternaspmm_probe_copy(vp(a), vp(b), nbytes, stream), 2 * nbytes)):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            fn()
        e1.record()
        torch.cuda.synchronize()
        out[name] = moved * 5 / (e0.elapsed_time(e1) * 1e-3) / 1e9
    out["read_copy_bytes"] = nbytes
    del a, b
    # the rate of the library's own largest stream: the bf16 LM head of the 2B shape, 128256 x 2560, one row of activations
    from ternainfer_amd.linear import lm_head
    w = torch.randn((128256, 2560), device="cuda", dtype=torch.bfloat16)
    x = torch.randn((1, 2560), device="cuda", dtype=torch.bfloat16)
    lg = torch.empty((1, 128256), device="cuda", dtype=torch.bfloat16)
    lm_head(x, w, lg)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        lm_head(x, w, lg)
    e1.record()
    torch.cuda.synchronize()
    out["lm_head_stream_GBps"] = w.numel() * 2 * 20 / (e0.elapsed_time(e1) * 1e-3) / 1e9
    del w, x, lg
    # device-wide synchronisation among co-resident workgroups (one per CU): what a persistent kernel would pay
    # between two dependent phases, to hold against the cost of a graph kernel node
    state = torch.zeros(lib.ternaspmm_probe_barrier_state_bytes() // 4, dtype=torch.int32, device="cuda")
    rounds, tag = 500, 1
    sync = {}
    for groups in (32, 64, 128, 256):
        best = None
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            rc = lib.ternaspmm_probe_barrier(vp(state), groups, rounds, tag, stream)
            e1.record()
            torch.cuda.synchronize()
            tag += rounds
            if rc != 0:
                break
            us = e0.elapsed_time(e1) * 1e3 / rounds
            best = us if best is None else min(best, us)
        sync[str(groups)] = best
    out["device_wide_sync_us_by_workgroups"] = sync
    out["device_wide_sync_timeouts"] = int(state[512].item())
    return out


# ------------------------------------------------------------------------------------------------ decode (configs[0], [1])
def layer_set_step(torch, lib, mats, layers, layout, m, steps, warmup):
    def step(stream):
        for layer in range(layers):
            for mt in mats:
                mt.launch(lib, layer, stream, layout, m)
    step(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))       # eager pass: code objects, outputs for the gate
    torch.cuda.synchronize()
    graph = capture(torch, step)
    # ---- the timed region: W warm-up replays, then exactly K steps between two synchronised events
    for _ in range(warmup):
        graph.replay()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(steps):
        graph.replay()
    ev1.record()
    torch.cuda.synchronize()
    return ev0.elapsed_time(ev1) / steps


def overlapped_layer_set(torch, lib, mats, layers, layout, m, steps, warmup):
    """The launches of the layer-set step with the dependence between them taken away: one stream per matrix shape inside
    the captured graph (fork at the start of a step, join at its end), every stream running its 30 launches back to back.
    A decoder cannot run like this -- each of its launches consumes the previous one's output -- so this is no throughput
    figure of the path; it shows what the same kernels on the same bytes reach once the per-launch latency chains
    overlap, i.e. how much of the distance to the HBM roofline is launch latency and how much is the kernels."""
    side = torch.cuda.Stream()
    branches = [torch.cuda.Stream() for _ in mats]
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            for br, mt in zip(branches, mats):
                br.wait_stream(side)
                with torch.cuda.stream(br):
                    handle = ctypes.c_void_p(br.cuda_stream)
                    for layer in range(layers):
                        mt.launch(lib, layer, handle, layout, m)
            for br in branches:
                side.wait_stream(br)
    torch.cuda.current_stream().wait_stream(side)
    return time_graph(torch, g, steps, warmup)


def config1_row(torch, T, lib, copies=400):
    """The literal single-matrix configuration: M = 8, K = N = 2560, P(0) = 0.45, one fp32 scale; cold = `copies`
    rotating weight copies (more than twice the last-level cache), hot = one copy."""
    from oracle import terna_oracle as O
    mt = Matrix("config1", 2560, 2560, 8, copies, 20260100, torch, T, p0=0.45)
    row = {"alg_bytes": mt.alg_bytes, "copies": copies}
    for layout in ("packed", "reference"):
        cold = capture(torch, lambda s: [mt.launch(lib, c, s, layout) for c in range(copies)])
        hot = capture(torch, lambda s: [mt.launch(lib, 0, s, layout) for _ in range(copies)])
        cold_us = time_graph(torch, cold, 5, 2) * 1e3 / copies
        hot_us = time_graph(torch, hot, 5, 2) * 1e3 / copies
        row[layout] = {"cold_us": cold_us, "cold_GBps": mt.alg_bytes / cold_us / 1e3, "cold_frac": mt.alg_bytes / cold_us / 1e3 / HBM_PEAK_GBPS,
                       "hot_us": hot_us, "hot_GBps": mt.alg_bytes / hot_us / 1e3}
        gold = O.spmm_bf16_golden(mt.x_bits, mt.w, mt.scale_host, 1)
        got = O.bf16_bits_to_f32(mt.out.cpu().numpy().view(np.uint16)).astype(np.float64)
        assert np.abs(got - gold).max() <= 1e-2 * np.abs(gold).max(), ("config1", layout)
    return row


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--m", type=int, default=8, help="activation rows per call (decode batch)")
    ap.add_argument("--layers", type=int, default=30, help="distinct weight copies per matrix")
    ap.add_argument("--workload", choices=["decode", "prefill", "model", "sweep", "midm"], default="decode",
                    help="decode: the headline small-M HBM-bound pass (plus, unless --no-extras, every other figure of the "
                         "path); prefill: the M>=256 MFMA-bound pass; model: random-init BitNet-2B-shaped "
                         "decoder, 128-token prompt + 256 greedy tokens; sweep: the sparsity / structure sweep at M=16; "
                         "midm: both kernel families at the batch sizes between decode and prefill")
    ap.add_argument("--batch", type=int, default=1, help="sequences decoded together (model workload)")
    ap.add_argument("--prompt-tokens", type=int, default=128,
                    help="prompt length of the model workload (configs[4]: 128, then 256 generated tokens; longer prompts: 128 "
                         "generated tokens; the attention kernels take caches of up to 8192 slots)")
    ap.add_argument("--act", choices=["int8", "bf16"], default=None,
                    help="activations into the ternary linears: int8 + per-row scale (the reference's SpBitLinear; "
                         "default of the model workload) or bf16 (default of the prefill workload)")
    ap.add_argument("--layout", choices=["packed", "reference"], default="packed",
                    help="packed: weights repacked once at load time to the library's P2 layout (bit-exact); "
                         "reference: kernels read the reference's compressed format directly")
    ap.add_argument("--no-prefetch", action="store_true",
                    help="model workload: no weight prefetch by the idle CUs of the attention launch")
    ap.add_argument("--no-chain", action="store_true",
                    help="model workload: the decode step without producer-side norm statistics (every linear re-derives them)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-per-shape", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="decode workload: only the headline step (no config1 / M sweep / prefill / model / calibration sections)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain 256 MiB device copy (calibrates FETCH_SIZE / WRITE_SIZE under rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    import ternainfer_amd as T
    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    lib = T._lib.load()
    torch.cuda.set_device(0)
    # The library's repack cache (on by default) gives reference-format callers the P2 kernels from the second sight of
    # a weight on.  Everything below that says "reference layout" times the kernels that read the reference format
    # itself, so the cache is off here; `drop_in_reference_format` switches it on for its own measurement.
    lib.ternaspmm_repack_cache_enable(0)

    if args.copy_probe:
        a = torch.empty(256 << 20, dtype=torch.int8, device="cuda")
        b = torch.ones(256 << 20, dtype=torch.int8, device="cuda")
        torch.cuda.synchronize()
        a.copy_(b)                                     # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
    if args.workload != "decode":
        runner = {"prefill": lambda: run_prefill(args, torch, T, lib), "model": lambda: run_model(args, torch),
                  "sweep": lambda: run_sweep(args, torch, T, lib), "midm": lambda: run_midm(args, torch, T, lib)}[args.workload]
        print(json.dumps(runner()))
        return

    t_start = time.perf_counter()
    mats = [Matrix(name, n, k, args.m, args.layers, 20260200 + 10 * j, torch, T)
            for j, (name, n, k) in enumerate(LAYER_SET)]
    step_bytes = args.layers * sum(mt.alg_bytes for mt in mats)
    launches_per_step = args.layers * len(mats)

    ms_per_step = layer_set_step(torch, lib, mats, args.layers, args.layout, args.m, args.steps, args.warmup)
    gbps = step_bytes / (ms_per_step * 1e-3) / 1e9
    launch_us = ms_per_step * 1e3 / launches_per_step
    default_workload = args.m == 8 and args.layers == 30 and args.layout == "packed"

    result = {
        "metric": METRIC,
        "value": gbps, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": (f"configs[1]: BitNet-b1.58-2B decode layer set (QKV 2560->3840, O 2560->2560, "
                                f"gate+up 2560->13824, down 6912->2560), M={args.m}, P(0)=0.40, bf16 activations, "
                                f"{args.layers} layers with distinct weight copies (cold stream), HIP-graph replay; weight layout: "
                                + ("P2, repacked once at load time from the reference format" if args.layout == "packed"
                                   else "reference format read directly")),
                   "m": args.m, "layers": args.layers, "layout": args.layout, "launches_per_step": launches_per_step,
                   "algorithmic_bytes_per_step": step_bytes},
        "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": gbps / HBM_PEAK_GBPS,
                     "traffic": TRAFFIC["bytes_per_launch"] if default_workload else None,
                     "traffic_source": TRAFFIC["source"] if default_workload else None,
                     "traffic_measured_at": TRAFFIC["measured_at"] if default_workload else None,
                     "kernel": ("terna_decode_chunk_kernel<bf16> / terna_decode_chunk4_kernel<bf16>" if args.layout == "packed" and args.m <= 16
                                else ("terna_decode_packed_kernel<bf16>" if args.layout == "packed" else "terna_decode_kernel<bf16>")),
                     "algorithmic_bytes_per_launch": step_bytes / launches_per_step,
                     "avg_launch_us": launch_us},
        "tokens_per_s_linear_layers_only": args.m / (ms_per_step * 1e-3) if args.layers == 30 else None,
    }

    # ---- per-shape detail: cold (rotating copies) and hot (one copy, cache resident)
    if not args.no_per_shape:
        shapes = {}
        for mt in mats:
            cold = capture(torch, lambda s, mt=mt: [mt.launch(lib, c, s, args.layout) for c in range(args.layers)])
            hot = capture(torch, lambda s, mt=mt: [mt.launch(lib, 0, s, args.layout) for _ in range(args.layers)])
            other = "reference" if args.layout == "packed" else "packed"
            alt = capture(torch, lambda s, mt=mt: [mt.launch(lib, c, s, other) for c in range(args.layers)])
            cold_us = time_graph(torch, cold, 20, 3) * 1e3 / args.layers
            hot_us = time_graph(torch, hot, 20, 3) * 1e3 / args.layers
            alt_us = time_graph(torch, alt, 20, 3) * 1e3 / args.layers
            shapes[f"{mt.name}_{mt.k}x{mt.n}"] = {
                "alg_bytes": mt.alg_bytes, "cold_us": cold_us, "cold_GBps": mt.alg_bytes / cold_us / 1e3,
                "cold_frac": mt.alg_bytes / cold_us / 1e3 / HBM_PEAK_GBPS,
                "hot_us": hot_us, "hot_GBps": mt.alg_bytes / hot_us / 1e3, f"cold_us_{other}_layout": alt_us,
                "tflops": 2.0 * mt.m * mt.n * mt.k / cold_us / 1e6}
        result["per_shape"] = shapes

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(mats, torch)

    if not args.no_extras:
        # the same layer set through the symbols an unmodified model.py binds (reference-format pointers), and at M = 1 / 16
        def as_figures(ms, what):
            return {"ms_per_step": ms, "GBps": step_bytes / (ms * 1e-3) / 1e9, "frac": step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                    "what": what}
        half = max(args.steps // 2, 5)
        result["reference_format_kernels"] = as_figures(
            layer_set_step(torch, lib, mats, args.layers, "reference", args.m, half, 2),
            "the same step through bitlinear_TernaSpMM_bf16 on reference-format pointers, repack cache off: the kernels that "
            "read the reference format directly")
        lib.ternaspmm_repack_cache_enable(1)
        for mt in mats:
            mt.out.fill_(-1)                             # poison: the leg's own launches must produce the checked outputs
        result["drop_in_reference_format"] = as_figures(
            layer_set_step(torch, lib, mats, args.layers, "reference", args.m, half, 2),
            "the same step through bitlinear_TernaSpMM_bf16 on reference-format pointers as an unmodified call site issues it "
            "(library defaults: every weight repacked once on first sight, every launch re-checks the copy's fingerprint)")
        result["drop_in_reference_format"]["parity_max_err_over_max_ref"] = golden_gate(mats, "drop-in leg")
        stats = (ctypes.c_longlong * 6)()
        lib.ternaspmm_repack_cache_stats(stats)
        result["drop_in_reference_format"]["repack_cache"] = {"copies": stats[0], "bytes": stats[1], "dropped_as_stale": stats[2]}
        assert stats[0] == args.layers * len(mats) and stats[2] == 0
        lib.ternaspmm_repack_cache_enable(0)
        lib.ternaspmm_repack_cache_clear()
        by_m = {}
        for m in (1, 16):
            ms = layer_set_step(torch, lib, mats, args.layers, args.layout, m, max(args.steps // 2, 5), 2)
            b = args.layers * sum(mt.bytes_at(m) for mt in mats)
            by_m[str(m)] = {"ms_per_step": ms, "GBps": b / (ms * 1e-3) / 1e9, "frac": b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                            "algorithmic_bytes_per_step": b}
        result["layer_set_by_m"] = by_m
        ms = overlapped_layer_set(torch, lib, mats, args.layers, args.layout, args.m, half, 2)
        result["launches_overlapped"] = as_figures(
            ms, "NOT a figure of the path: the same launches with the dependence between them removed (one stream per matrix shape "
                "inside the graph, four chains of 30 launches side by side) -- what the kernels reach on these bytes when the "
                "per-launch latency chains overlap; a decoder's launches depend on each other and cannot run like this")
        del mats
        torch.cuda.empty_cache()
        result["config1"] = config1_row(torch, T, lib)
        torch.cuda.empty_cache()
        ps = PrefillSet(torch, T, [2048])
        result["prefill_m2048"] = {act: prefill_figures(ps, lib, act, 2048, 50, 10) for act in ("bf16", "int8")}
        del ps
        torch.cuda.empty_cache()
        model = None
        md = {}
        for batch in (1, 8):
            md[f"batch{batch}"], model = measure_model(torch, batch, "int8", True, model=model)
        # the same model far into a long context: one sequence, 1920-token prompt, 128 tokens (cache of 2048 slots)
        md["batch1_context2048"], model = measure_model(torch, 1, "int8", True, gen_tokens=128, model=model, prompt_tokens=1920)
        result["model_decode"] = md
        del model
        torch.cuda.empty_cache()
        result["calibration"] = calibration(torch, lib)
        result["bench_wall_s"] = time.perf_counter() - t_start

    print(json.dumps(result))


if __name__ == "__main__":
    main()
