"""Measurement harness: a BitNet-b1.58-2B-shaped decoder whose linear layers run through TernaSpMM.

This is NOT a port of the reference's transformer (model.py:155-471); it exists so that the
2B-shape decode tokens/s of the benchmark configuration can be measured with every ternary linear
going through libternaspmm.so.  It keeps the reference's block structure -- fused wqkv / w13,
attention and FFN sub-norms, squared-ReLU gating, tied bf16 LM head (model.py:198-239, 277-282,
323-335, 367) -- and, like the reference's SpBitLinear (model.py:120-133), quantises activations
per row to int8 in front of every ternary linear.  The residual adds, the four norms, the gate and
that quantisation run as the library's fused prologue kernels (one launch in front of each
linear); RoPE + KV-cache write, single-token attention, the multi-token attention of the prompt
pass, the LM head of a decode step and greedy sampling are library kernels too (the prompt pass projects
its last rows through the LM head with a PyTorch-ROCm matmul); the prompt pass and one decode step are
each captured in a HIP graph, as generate.py:204-224 does for the decode step.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Optional

import torch
from torch.nn import functional as F

from . import _lib
from .linear import (EPILOGUE_GATE, EPILOGUE_RESIDUAL, argmax_rows, attention_merge_rmsnorm_linear_packed, attention_merge_rmsnorm_quant, fused_linear, get_global_workspace, greedy_step,
                     greedy_step_state, interleave_gate_up, lm_head, quant_from_stats, quant_input, row_stats, relu2_mul_rmsnorm_linear_packed, relu2_mul_rmsnorm_quant, step_inputs,
                     repack_weight, rmsnorm_linear_packed, rmsnorm_quant)


@dataclass
class ModelArgs:                      # model.py:23-34
    dim: int = 2560
    n_layers: int = 30
    n_heads: int = 20
    n_kv_heads: int = 5
    vocab_size: int = 128256
    ffn_dim: int = 6912
    norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_adjacent: bool = True        # pairs (2j, 2j+1), rope_padded's default (model.py:221-229); False = (j, j + D/2)

    @property
    def head_dim(self) -> int:
        return self.dim // self.n_heads


def _p(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def random_p2_weight(n: int, k: int, p_zero: float, gen: torch.Generator, device="cuda") -> torch.Tensor:
    """Random ternary [n, k] matrix, generated on the device directly in the library's P2 layout
    (uint32 [n/16][k/64][64], see csrc/packed_common.h): P(0) = p_zero, signs balanced."""
    u = torch.rand((n // 16, 16, k // 64, 4, 16), generator=gen, device=device)           # band, i, gk, g, q
    neg = torch.rand(u.shape, generator=gen, device=device) < 0.5
    code = (u >= p_zero).to(torch.int64) | ((u >= p_zero) & neg).to(torch.int64) << 1
    j = torch.arange(16, device=device)
    shift = 8 * (j & 3) + 2 * (j >> 2)
    words = (code << shift).sum(dim=-1)                                                     # band, i, gk, g
    words = words.permute(0, 2, 1, 3).contiguous().view(n // 16, k // 64, 64)
    return (words - ((words >> 31) << 32)).to(torch.int32)                                  # same 32 bits, signed storage


class TernaryLinear:
    """One ternary matrix in P2 layout + its weight-group scales; forward = TernaSpMM."""

    def __init__(self, in_features: int, out_features: int, packed: torch.Tensor, weight_scale: torch.Tensor,
                 act: str = "int8"):
        self.k, self.n = in_features, out_features
        self.packed = packed
        self.ws = weight_scale.to(torch.bfloat16).contiguous()                  # bf16[4], zero padded (convert_TernaInfer.py:176-194)
        self.ws_num = int((self.ws != 0).sum().item())
        self.scale_f32 = self.ws.float().contiguous()
        self.act = act
        self.lib = _lib.load()

    def quantised(self, xq: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
        """int8 activations [M, K] + per-row scale bf16 [M] (as the fused prologue kernels write them)."""
        m = xq.shape[0]
        out = torch.empty((m, self.n), dtype=torch.bfloat16, device=xq.device)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        work = get_global_workspace(xq.device) if m > 64 else None              # large M: room for split-K partial sums
        self.lib.bitlinear_TernaSpMM_packed_ws(_p(xq), _p(self.packed), _p(out), _p(s), _p(self.ws), self.ws_num,
                                               m, self.n, self.k, 0, _p(work), work.numel() if work is not None else 0, stream)
        return out

    def dense(self, x: torch.Tensor) -> torch.Tensor:
        """bf16 activations [M, K]."""
        m = x.shape[0]
        out = torch.empty((m, self.n), dtype=torch.bfloat16, device=x.device)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        work = get_global_workspace(x.device) if m > 64 else None
        self.lib.bitlinear_TernaSpMM_bf16_packed_ws(_p(x.contiguous()), _p(self.packed), _p(out), _p(self.scale_f32),
                                                    self.ws_num, m, self.n, self.k, 0, _p(work),
                                                    work.numel() if work is not None else 0, stream)
        return out

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        if self.act == "int8":                # model.py:120-133
            xq, s = quant_input(x)
            return self.quantised(xq, s.reshape(-1).contiguous())
        return self.dense(x)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """fp32 inside, one rounding to the input's dtype (the fused kernels compute the same)."""
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(x.dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, adjacent: bool = True) -> torch.Tensor:
    """x [B, H, T, D]; cos/sin broadcastable to [B, H, T, D/2], fp32; pair j = (x[2j], x[2j+1]) when
    `adjacent`, else (x[j], x[j + D/2])."""
    xf = x.float()
    if adjacent:
        x1, x2 = xf[..., 0::2], xf[..., 1::2]
        return torch.stack([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1).flatten(-2).to(x.dtype)
    x1, x2 = xf.chunk(2, dim=-1)
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1).to(x.dtype)


KERNEL_ATTENTION = object()    # in place of a mask: several new tokens, attention by ternaspmm_prefill_attention


class Block:
    # forward_chain: up to this many rows the O projection takes the sub-norm's statistics inside; above, the norm kernel
    # and the O projection on its quantised rows (measured: 4 sequences 3917 against 3769 tokens/s, 5 sequences 4285
    # against 4343, 8 sequences 6708 against 6849)
    o_norm_rows = 4
    attention_stats_chain = True   # the same for 2 .. o_norm_rows sequences, consumed by the O projection's STATS prologue (+1 - 1.6 %)
    attention_stats = True         # ... and the unsplit attention launch leaves the sub-norm's partial statistics (see forward_chain)
    merge_quant = True             # forward_chain, several sequences, deferred attention merge: the merge launch also norms and quantises
    chain_down_rows = 2            # forward_chain: up to this many rows the down projection (K = ffn_dim) norms + quantises inside its launch

    def __init__(self, args: ModelArgs, gen: Optional[torch.Generator], act: str, p_zero: float = 0.40):
        self.args = args
        self.act = act
        self.fused = True          # norms / gate / activation quantisation through the fused prologue kernels
        self.prefetch = None       # (pointers, sizes, unit sizes, count): see Transformer.enable_prefetch
        self.capture = None        # a list: forward_chain appends (name, xq, s, raw output) of each of its four linears
        self.w13_interleaved = None
        if gen is None:            # filled in by from_checkpoint
            return
        d, hd = args.dim, args.head_dim
        qkv_n = (args.n_heads + 2 * args.n_kv_heads) * hd
        bf = lambda v: torch.tensor(v + [0.0] * (4 - len(v)), dtype=torch.bfloat16, device="cuda")
        sc = lambda: float(torch.empty(1).uniform_(0.5, 2.0, generator=gen_cpu))
        gen_cpu = torch.Generator().manual_seed(int(torch.randint(0, 2 ** 31, (1,), generator=gen, device="cuda").item()))
        self.wqkv = TernaryLinear(d, qkv_n, random_p2_weight(qkv_n, d, p_zero, gen), bf([sc(), sc(), sc()]), act)
        self.wo = TernaryLinear(args.n_heads * hd, d, random_p2_weight(d, args.n_heads * hd, p_zero, gen), bf([sc()]), act)
        self.w13 = TernaryLinear(d, 2 * args.ffn_dim, random_p2_weight(2 * args.ffn_dim, d, p_zero, gen), bf([sc(), sc()]), act)
        self.w2 = TernaryLinear(args.ffn_dim, d, random_p2_weight(d, args.ffn_dim, p_zero, gen), bf([sc()]), act)
        ones = lambda n: torch.ones(n, dtype=torch.bfloat16, device="cuda")
        self.attention_norm, self.ffn_norm = ones(d), ones(d)
        self.attn_sub_norm, self.ffn_sub_norm = ones(d), ones(args.ffn_dim)

    @classmethod
    def from_checkpoint(cls, args: ModelArgs, dic: dict, layer_prefix: str, act: str = "int8") -> "Block":
        """One block from the merged checkpoint dictionary (keys as model.py:110-116, 195, 275, 320-321):
        the four format tensors of each linear are uploaded, repacked to P2 once and dropped."""
        blk = cls(args, None, act)
        d, hd = args.dim, args.head_dim
        shapes = {"attention.wqkv": (d, (args.n_heads + 2 * args.n_kv_heads) * hd), "attention.wo": (args.n_heads * hd, d),
                  "feed_forward.w13": (d, 2 * args.ffn_dim), "feed_forward.w2": (args.ffn_dim, d)}
        for name, (k, n) in shapes.items():
            key = f"{layer_prefix}.{name}"
            parts = [dic[key + ".weight" + suffix].cuda()
                     for suffix in ("_compressed_val", "_TileOffsets_global", "_TileOffsets_median", "_bitmap")]
            packed = repack_weight(*parts, n, k)
            torch.cuda.synchronize()       # the format tensors are released below; the repack must have read them
            setattr(blk, name.split(".")[1], TernaryLinear(k, n, packed, dic[key + ".weight_scale"].cuda(), act))
        norm = lambda name: dic[f"{layer_prefix}.{name}.weight"].to(device="cuda", dtype=torch.bfloat16).contiguous()
        blk.attention_norm, blk.ffn_norm = norm("attention_norm"), norm("ffn_norm")
        blk.attn_sub_norm, blk.ffn_sub_norm = norm("attention.attn_sub_norm"), norm("feed_forward.ffn_sub_norm")
        return blk

    def _norm_linear(self, lin, x, weight, residual=None, glu=False, name=None):
        """[x + residual | relu(x1)^2 * x3] -> RMSNorm -> lin.  Returns (lin output, x + residual).  With `capture` set the
        quantised activations go through memory (norm kernel + linear, never the one-launch form) and are recorded."""
        eps = self.args.norm_eps
        if not self.fused:
            if glu:
                x1, x3 = x.chunk(2, dim=-1)
                h = F.relu(x1) ** 2 * x3
            else:
                h = x if residual is None else x + residual
            return lin(rms_norm(h, weight, eps)), h
        cap = self.capture if self.act == "int8" else None
        if glu:
            if self.act == "int8":
                if x.shape[0] <= 4 and cap is None:
                    return relu2_mul_rmsnorm_linear_packed(x, weight, eps, lin.packed, lin.ws, lin.ws_num, lin.n), None
                xq, s = relu2_mul_rmsnorm_quant(x, weight, eps)
                out = lin.quantised(xq, s)
                if cap is not None:
                    cap.append((name, xq, s, out))
                return out, None
            return lin.dense(relu2_mul_rmsnorm_quant(x, weight, eps, quant=False)), None
        if self.act == "int8":
            if x.shape[0] <= 8 and cap is None:   # decode step: prologue and linear in one launch where that is faster
                return rmsnorm_linear_packed(x, weight, eps, lin.packed, lin.ws, lin.ws_num, lin.n, residual=residual)
            xq, s, h = rmsnorm_quant(x, weight, eps, residual=residual)
            out = lin.quantised(xq, s)
            if cap is not None:
                cap.append((name, xq, s, out))
            return out, h
        y, h = rmsnorm_quant(x, weight, eps, residual=residual, quant=False)
        return lin.dense(y), h

    def gate_up_interleaved(self):
        """The gate+up matrix with the bands of w1 and w3 interleaved (made once): what the gate epilogue reads."""
        if self.w13_interleaved is None:
            self.w13_interleaved = interleave_gate_up(self.w13.packed, self.w13.n, self.w13.k)
        return self.w13_interleaved

    def forward_chain(self, x, stats, cache_k, cache_v, pos_idx, cos, sin, attn_ws, next_norm, split=False):
        """One new token per sequence (up to 16 sequences), the linears chained through producer-side norm statistics:
        `x` is the residual stream INCLUDING the previous block's FFN output and `stats` its partials under this block's
        attention_norm (None: the first block, which takes them inside).  Every linear's epilogue leaves what the next
        launch needs: the O projection adds the stream and leaves the ffn_norm partials, gate+up leaves
        relu(x1)^2 * x3 with the ffn_sub_norm partials, the down projection adds the stream again and leaves the
        partials under `next_norm` (the next block's attention_norm).  Returns (stream, partials).
        `split`: the producers are the same, but the norm + quantisation in front of QKV, gate+up and the down projection
        is a launch of its own from the partials (quant_from_stats: element-wise, no reduction over the row) and the
        linears take the quantised rows -- for row counts at which every workgroup repeating that work costs more."""
        a = self.args
        bsz = cache_k.shape[0]
        lib = self.wqkv.lib
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        per_seq = int(pos_idx.dim() == 2)
        cap = self.capture
        pub = cap is not None

        def note(name, r):
            if pub:
                cap.append((name, r[3], r[4], r[2] if r[2] is not None else r[0]))

        if split:
            xq, s = quant_from_stats(x, stats, self.attention_norm, a.norm_eps) if stats is not None else rmsnorm_quant(x, self.attention_norm, a.norm_eps)[:2]
            qkv = self.wqkv.quantised(xq, s)
            if pub:
                cap.append(("wqkv", xq, s, qkv))
        elif stats is None and not pub:
            qkv, _ = rmsnorm_linear_packed(x, self.attention_norm, a.norm_eps, self.wqkv.packed, self.wqkv.ws, self.wqkv.ws_num, self.wqkv.n)
        else:
            if stats is None:                       # (recording: the first block's statistics as a launch of their own)
                stats = row_stats(x, self.attention_norm)
            r = fused_linear(x, self.attention_norm, a.norm_eps, self.wqkv.packed, self.wqkv.ws, self.wqkv.ws_num, self.wqkv.n, self.wqkv.k,
                             stats=stats, publish=pub)
            note("wqkv", r)
            qkv = r[0]
        deferred = isinstance(attn_ws, tuple)
        o_kw = dict(epilogue=EPILOGUE_RESIDUAL, residual=x, next_norm_weight=self.ffn_norm, want_raw=pub, publish=pub)
        if deferred:
            partial, splits = attn_ws
            # (weights of the next launches through the caches meanwhile: only next to a short attention -- with caches of
            # 1528 slots the prefetch cost 2 % of the step, at 728 slots it gains 0.5 %)
            pf = self.prefetch if split and self.prefetch is not None and cache_k.shape[2] <= 1024 else (None, None, None, 0)
            lib.ternaspmm_rope_decode_attention_partial(
                _p(qkv), _p(cos), _p(sin), _p(pos_idx), per_seq, _p(cache_k), _p(cache_v), _p(partial), splits, bsz, a.n_heads,
                a.n_kv_heads, a.head_dim, cache_k.shape[2], a.head_dim ** -0.5, int(a.rope_adjacent), *pf, stream)
            r = None
            if split or (bsz > 1 and self.merge_quant):
                # merge + sub-norm + quantisation once per sequence, then the O projection on the quantised rows
                mq = attention_merge_rmsnorm_quant(partial, splits, a.n_heads, a.head_dim, self.attn_sub_norm, a.norm_eps, bsz, want_output=pub)
                if mq is not None:
                    if pub:
                        cap.append(("attention", None, None, mq[2]))
                    r = fused_linear(mq[0], None, a.norm_eps, self.wo.packed, self.wo.ws, self.wo.ws_num, self.wo.n, self.wo.k, quantised=mq[1],
                                     epilogue=EPILOGUE_RESIDUAL, residual=x, next_norm_weight=self.ffn_norm, want_raw=pub)
                    if r is not None:
                        r = (r[0], r[1], r[2], mq[0], mq[1])
            elif bsz == 1:
                r = fused_linear(partial, self.attn_sub_norm, a.norm_eps, self.wo.packed, self.wo.ws, self.wo.ws_num, self.wo.n, self.wo.k,
                                 attention=(splits, a.head_dim), **o_kw)
            if r is None:
                o = torch.empty((bsz, a.n_heads * a.head_dim), dtype=torch.bfloat16, device=x.device)
                lib.ternaspmm_attention_merge(_p(partial), splits, _p(o), bsz, a.n_heads, a.head_dim, stream)
                r = fused_linear(o, self.attn_sub_norm, a.norm_eps, self.wo.packed, self.wo.ws, self.wo.ws_num, self.wo.n, self.wo.k, **o_kw)
        else:
            o = torch.empty((bsz, a.n_heads * a.head_dim), dtype=torch.bfloat16, device=x.device)
            o_stats = None
            if self.prefetch is not None:
                ptrs, sizes, units, count = self.prefetch
                lib.ternaspmm_rope_decode_attention_prefetch(
                    _p(qkv), _p(cos), _p(sin), _p(pos_idx), per_seq, _p(cache_k), _p(cache_v), _p(o), bsz, a.n_heads, a.n_kv_heads,
                    a.head_dim, cache_k.shape[2], a.head_dim ** -0.5, int(a.rope_adjacent), _p(attn_ws), ptrs, sizes, units,
                    count, stream)
            elif (bsz > self.o_norm_rows or (bsz > 1 and self.attention_stats_chain)) and self.attention_stats:
                # the unsplit launch also leaves the sub-norm's partial statistics per head: the quantised rows of the O
                # projection then come from the element-wise launch instead of the norm kernel
                o_stats = torch.empty((bsz, a.n_heads, 2), dtype=torch.float32, device=x.device)
                if lib.ternaspmm_rope_decode_attention_stats(_p(qkv), _p(cos), _p(sin), _p(pos_idx), per_seq, _p(cache_k), _p(cache_v), _p(o),
                                                             bsz, a.n_heads, a.n_kv_heads, a.head_dim, cache_k.shape[2], a.head_dim ** -0.5,
                                                             int(a.rope_adjacent), _p(self.attn_sub_norm), _p(o_stats), stream) != a.n_heads:
                    raise RuntimeError("ternaspmm_rope_decode_attention_stats refused the launch")
            else:
                lib.ternaspmm_rope_decode_attention(_p(qkv), _p(cos), _p(sin), _p(pos_idx), per_seq, _p(cache_k), _p(cache_v), _p(o),
                                                    bsz, a.n_heads, a.n_kv_heads, a.head_dim, cache_k.shape[2],
                                                    a.head_dim ** -0.5, int(a.rope_adjacent), _p(attn_ws), stream)
            if pub:
                cap.append(("attention", None, None, o))
            r = None
            if bsz <= self.o_norm_rows:          # the sub-norm's statistics taken inside the O projection (or given by the attention)
                r = fused_linear(o, self.attn_sub_norm, a.norm_eps, self.wo.packed, self.wo.ws, self.wo.ws_num, self.wo.n, self.wo.k,
                                 stats=o_stats, **o_kw)
            if r is None:                        # more rows: the norm kernel (or the quantise launch), then the O projection on quantised rows
                if o_stats is not None:
                    xq, s = quant_from_stats(o, o_stats, self.attn_sub_norm, a.norm_eps)
                else:
                    xq, s, _ = rmsnorm_quant(o, self.attn_sub_norm, a.norm_eps)
                r = fused_linear(xq, None, a.norm_eps, self.wo.packed, self.wo.ws, self.wo.ws_num, self.wo.n, self.wo.k, quantised=s,
                                 epilogue=EPILOGUE_RESIDUAL, residual=x, next_norm_weight=self.ffn_norm, want_raw=pub)
                r = (r[0], r[1], r[2], xq, s)
        note("wo", r)
        h, h_stats = r[0], r[1]
        if split:
            xq, s = quant_from_stats(h, h_stats, self.ffn_norm, a.norm_eps)
            r = fused_linear(xq, None, a.norm_eps, self.gate_up_interleaved(), self.w13.ws, self.w13.ws_num, self.w13.n, self.w13.k,
                             quantised=s, epilogue=EPILOGUE_GATE, next_norm_weight=self.ffn_sub_norm)
            r = (r[0], r[1], None, xq, s)
        else:
            r = fused_linear(h, self.ffn_norm, a.norm_eps, self.gate_up_interleaved(), self.w13.ws, self.w13.ws_num, self.w13.n, self.w13.k,
                             stats=h_stats, epilogue=EPILOGUE_GATE, next_norm_weight=self.ffn_sub_norm, publish=pub)
        note("w13", r)
        inner, inner_stats = r[0], r[1]
        if split or bsz > self.chain_down_rows:
            # K = 6912: from three rows on every workgroup repeating the norm + quantisation of the whole block costs more than
            # one launch that does it once (measured: 3 sequences 2972 -> 3031 tokens/s, 4 3976 -> 4004; 2 sequences 2094 against 2082)
            xq, s = quant_from_stats(inner, inner_stats, self.ffn_sub_norm, a.norm_eps)
            r = fused_linear(xq, None, a.norm_eps, self.w2.packed, self.w2.ws, self.w2.ws_num, self.w2.n, self.w2.k, quantised=s,
                             epilogue=EPILOGUE_RESIDUAL, residual=h, next_norm_weight=next_norm, want_raw=pub)
            r = (r[0], r[1], r[2], xq, s)
        else:
            r = fused_linear(inner, self.ffn_sub_norm, a.norm_eps, self.w2.packed, self.w2.ws, self.w2.ws_num, self.w2.n, self.w2.k,
                             stats=inner_stats, epilogue=EPILOGUE_RESIDUAL, residual=h, next_norm_weight=next_norm, want_raw=pub, publish=pub)
        note("w2", r)
        return r[0], r[1]

    def forward(self, x, pending, cache_k, cache_v, pos_idx, cos, sin, mask, attn_ws=None):
        """x [B*T, dim] (T new tokens per sequence) and `pending`, the previous block's FFN output that
        has not been added to the stream yet (None for the first block): the add is part of this
        block's first fused kernel.  cache_* [B, n_kv, S, hd]; pos_idx int64 [T] cache slots shared by the
        sequences, or [B, T] with cos / sin [B*T, hd/2]: every sequence at its own positions (generate.py:253-262).
        Returns (stream, pending) for the next block."""
        a = self.args
        bsz = cache_k.shape[0]
        t = x.shape[0] // bsz
        per_seq = int(pos_idx.dim() == 2)
        qkv, x = self._norm_linear(self.wqkv, x, self.attention_norm, residual=pending, name="wqkv")
        rep = a.n_heads // a.n_kv_heads
        one_token = mask is None           # the caller's rule: fused, one new token, a head size the kernel has
        deferred = one_token and isinstance(attn_ws, tuple)
        if deferred:
            # the cache prefix of every head split over several workgroups that leave partial results; the O
            # projection's prologue merges them (one sequence; else a merge launch): the launch boundary is the synchronisation
            lib = self.wqkv.lib
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            # (no prefetch regions here: this launch is shorter than the prefetch of the following weights would be --
            # measured with them 1005 - 1125 us per step against 960 without and 971 for the unsplit launch that prefetches)
            partial, splits = attn_ws
            lib.ternaspmm_rope_decode_attention_partial(
                _p(qkv), _p(cos), _p(sin), _p(pos_idx), per_seq, _p(cache_k), _p(cache_v), _p(partial), splits, bsz, a.n_heads,
                a.n_kv_heads, a.head_dim, cache_k.shape[2], a.head_dim ** -0.5, int(a.rope_adjacent), None, None, None, 0,
                stream)
        elif one_token:                     # RoPE, cache write and attention over the cache prefix: one launch
            lib = self.wqkv.lib
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            o = torch.empty((bsz, a.n_heads * a.head_dim), dtype=torch.bfloat16, device=x.device)
            if self.prefetch is not None:
                # the attention launch occupies one CU per head: extra workgroups of the same launch pull the
                # weights of the launches that follow through the caches meanwhile
                ptrs, sizes, units, count = self.prefetch
                lib.ternaspmm_rope_decode_attention_prefetch(
                    _p(qkv), _p(cos), _p(sin), _p(pos_idx), per_seq, _p(cache_k), _p(cache_v), _p(o), bsz, a.n_heads, a.n_kv_heads,
                    a.head_dim, cache_k.shape[2], a.head_dim ** -0.5, int(a.rope_adjacent), _p(attn_ws), ptrs, sizes, units,
                    count, stream)
            else:
                lib.ternaspmm_rope_decode_attention(_p(qkv), _p(cos), _p(sin), _p(pos_idx), per_seq, _p(cache_k), _p(cache_v), _p(o),
                                                    bsz, a.n_heads, a.n_kv_heads, a.head_dim, cache_k.shape[2],
                                                    a.head_dim ** -0.5, int(a.rope_adjacent), _p(attn_ws), stream)
        elif self.fused:
            lib = self.wqkv.lib
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            q = torch.empty((bsz, a.n_heads, t, a.head_dim), dtype=torch.bfloat16, device=x.device)
            lib.ternaspmm_rope_kv_store(_p(qkv), _p(cos), _p(sin), _p(pos_idx), per_seq, _p(q), _p(cache_k), _p(cache_v),
                                        bsz, t, a.n_heads, a.n_kv_heads, a.head_dim, cache_k.shape[2],
                                        int(a.rope_adjacent), stream)
            if mask is KERNEL_ATTENTION:    # the prompt pass: the library's multi-token attention over the cache
                o = torch.empty((bsz * t, a.n_heads * a.head_dim), dtype=torch.bfloat16, device=x.device)
                lib.ternaspmm_prefill_attention(_p(q), _p(cache_k), _p(cache_v), _p(pos_idx), per_seq, _p(o), bsz, t, a.n_heads,
                                                a.n_kv_heads, a.head_dim, cache_k.shape[2], a.head_dim ** -0.5, stream)
        else:
            qkv = qkv.view(bsz, t, a.n_heads + 2 * a.n_kv_heads, a.head_dim).transpose(1, 2)
            q, k, v = qkv[:, :a.n_heads], qkv[:, a.n_heads:a.n_heads + a.n_kv_heads], qkv[:, a.n_heads + a.n_kv_heads:]
            if per_seq:
                cs, sn = cos.view(bsz, 1, t, -1), sin.view(bsz, 1, t, -1)
            else:
                cs, sn = cos[None, None], sin[None, None]
            q = apply_rope(q, cs, sn, a.rope_adjacent)
            k = apply_rope(k, cs, sn, a.rope_adjacent)
            if per_seq:
                for b in range(bsz):
                    cache_k[b].index_copy_(1, pos_idx[b], k[b])
                    cache_v[b].index_copy_(1, pos_idx[b], v[b])
            else:
                cache_k.index_copy_(2, pos_idx, k)
                cache_v.index_copy_(2, pos_idx, v)
        if not one_token and mask is not KERNEL_ATTENTION:
            kk = cache_k.repeat_interleave(rep, dim=1)
            vv = cache_v.repeat_interleave(rep, dim=1)
            o = F.scaled_dot_product_attention(q, kk, vv, attn_mask=mask)
            o = o.transpose(1, 2).reshape(bsz * t, a.n_heads * a.head_dim)
        if deferred:
            attn = attention_merge_rmsnorm_linear_packed(partial, splits, a.n_heads, a.head_dim, self.attn_sub_norm, a.norm_eps,
                                                         self.wo.packed, self.wo.ws, self.wo.ws_num, self.wo.n, sequences=bsz)
            assert attn.shape[0] == bsz
        else:
            if self.capture is not None:
                self.capture.append(("attention", None, None, o))
            attn, _ = self._norm_linear(self.wo, o.contiguous(), self.attn_sub_norm, name="wo")
        x13, x = self._norm_linear(self.w13, x, self.ffn_norm, residual=attn, name="w13")
        ffn, _ = self._norm_linear(self.w2, x13, self.ffn_sub_norm, glu=True, name="w2")
        return x, ffn


class Transformer:
    """Random-init decoder; `act` selects int8-quantised (reference semantics) or bf16 activations."""

    # Up to this many sequences a one-token step chains its linears with the norm + quantisation inside the consuming
    # linear (Block.forward_chain).  Every workgroup of such a linear normalises and quantises the whole activation matrix
    # again, and one of its waves per row only adds up partials; from five rows on that costs more than a launch that does
    # it once (measured at 5, 6 and 8 rows).
    chain_rows = 4
    # Above that, up to this many sequences, the producing epilogues stay (residual add, gate, partial statistics) and a
    # small element-wise launch forms the quantised rows from the partials (Block.forward_chain, split): lighter than the
    # norm kernels, which reduce over the row twice, and the gate+up launch writes F columns instead of 2F.
    split_rows = 16
    # Cache slots from which on a chained step of 2 .. chain_rows sequences splits its attention and leaves the merge to a
    # launch of its own (measured, 4 sequences: 428 slots 1.041 ms per step unsplit against 1.115, 728 slots 1.154 against 1.120)
    defer_above = 640

    def __init__(self, args: ModelArgs, seed: int = 0, act: str = "int8", p_zero: float = 0.40):
        gen = torch.Generator(device="cuda").manual_seed(seed)
        self.args = args
        self.tok_embeddings = (torch.randn((args.vocab_size, args.dim), generator=gen, device="cuda") * 0.02).to(torch.bfloat16)
        self.layers: List[Block] = [Block(args, gen, act, p_zero) for _ in range(args.n_layers)]
        self.norm = torch.ones(args.dim, dtype=torch.bfloat16, device="cuda")

    @classmethod
    def from_checkpoint(cls, args: ModelArgs, dic: dict, act: str = "int8") -> "Transformer":
        """The model of a converted checkpoint: `dic` is the ternary and the non-ternary file merged
        (generate.py:69-71; ternainfer_amd.convert_utils.load_checkpoint)."""
        model = cls.__new__(cls)
        model.args = args
        model.tok_embeddings = dic["tok_embeddings.weight"].to(device="cuda", dtype=torch.bfloat16).contiguous()
        model.layers = [Block.from_checkpoint(args, dic, f"layers.{n}", act) for n in range(args.n_layers)]
        model.norm = dic["norm.weight"].to(device="cuda", dtype=torch.bfloat16).contiguous()
        return model

    def pack_norm_weights(self) -> None:
        """All norm weights of the model in one buffer, in the order the decode step reads them, so that a block's
        attention launch can prefetch the ones of the launches that follow as one region."""
        names = ("attention_norm", "attn_sub_norm", "ffn_norm", "ffn_sub_norm")
        total = sum(getattr(blk, nm).numel() for blk in self.layers for nm in names)
        buf = torch.empty(total, dtype=torch.bfloat16, device=self.norm.device)
        off = 0
        for blk in self.layers:
            blk.norm_offsets = {}
            for nm in names:
                w = getattr(blk, nm)
                view = buf[off:off + w.numel()]
                view.copy_(w)
                setattr(blk, nm, view)
                blk.norm_offsets[nm] = off
                off += w.numel()
        self.norm_buffer = buf

    def enable_prefetch(self, on: bool = True, which=("wo", "w13", "w2", "next_wqkv", "norms")) -> None:
        """Single-token steps: while a block's attention runs (one workgroup per head), extra workgroups of that
        launch prefetch the weights of its O, gate+up and down projections and of the next block's QKV projection
        (`which` picks among them).  Measured on MI355X with the unsplit attention launch: +6 % tokens/s at batch 1 with
        all four.  With the step as it is now -- one sequence runs the split attention, which passes no regions -- it pays
        for two sequences (+1 %); from three on the step is 1.4 - 1.7 % faster without, and where few CUs are left idle the
        prefetching workgroups become the launch's critical path (nine to eleven sequences: 10 - 20 % slower)."""
        for n, blk in enumerate(self.layers):
            if not on:
                blk.prefetch = None
                continue
            unit = lambda lin, bands: bands * (lin.k // 64) * 256        # what one consuming workgroup reads
            regions = []
            if "wo" in which:
                regions.append((blk.wo.packed, unit(blk.wo, 1)))
            if "w13" in which:
                regions.append((blk.w13.packed, unit(blk.w13, 4)))
            if "w2" in which:
                regions.append((blk.w2.packed, unit(blk.w2, 1)))
            if "next_wqkv" in which and n + 1 < len(self.layers):
                nxt = self.layers[n + 1].wqkv
                regions.append((nxt.packed, unit(nxt, 1)))
            if "norms" in which:
                if getattr(self, "norm_buffer", None) is None:
                    self.pack_norm_weights()
                # attn_sub_norm, ffn_norm, ffn_sub_norm of this block and attention_norm of the next: contiguous
                first = blk.norm_offsets["attn_sub_norm"]
                last = self.layers[n + 1].norm_offsets["attn_sub_norm"] if n + 1 < len(self.layers) else self.norm_buffer.numel()
                first -= first % 8                                        # 16-byte aligned start
                regions.append((self.norm_buffer[first:last], 0))         # unit 0: every XCD fetches it whole
            count = len(regions)
            ptrs = (ctypes.c_void_p * count)(*[w.data_ptr() for w, _ in regions])
            sizes = (ctypes.c_longlong * count)(*[w.numel() * w.element_size() for w, _ in regions])
            units = (ctypes.c_longlong * count)(*[u for _, u in regions])
            blk.prefetch = (ptrs, sizes, units, count)

    def chain_supported(self) -> bool:
        """Shapes ternaspmm_fused_linear takes for every linear of a block (see include/ternaspmm.h)."""
        a = self.args
        qd = a.n_heads * a.head_dim
        return (a.dim % 64 == 0 and qd % 64 == 0 and a.ffn_dim % 64 == 0 and a.dim <= 2560 and qd <= 2560 and a.ffn_dim <= 7168
                and a.dim // 16 <= 448 and a.ffn_dim // 16 <= 448)

    def rope_tables(self, max_seq: int, dev):
        """cos / sin of every (cache slot, rotary pair): fp32 [max_seq, 2, head_dim / 2] (cos row, sin row), built
        once per length; one gather then fetches both rows of a position."""
        key = (max_seq, str(dev))
        tables = getattr(self, "_rope_tables", None)
        if tables is None or tables[0] != key:
            a = self.args
            inv = 1.0 / (a.rope_theta ** (torch.arange(0, a.head_dim, 2, device=dev, dtype=torch.float32) / a.head_dim))
            ang = torch.arange(max_seq, device=dev, dtype=torch.float32)[:, None] * inv[None, :]
            self._rope_tables = tables = (key, torch.stack([ang.cos(), ang.sin()], dim=1).contiguous())
        return tables[1]

    def attention_partial(self, bsz: int, max_seq: int, single_split: bool = False):
        """(buffer, splits) for the decode step whose attention leaves the merge of its splits to the consumer of its
        output (one sequence: the O projection's prologue; more: a merge launch), or None when that form does not apply
        (one split recommended and not `single_split`; `deferred_attention_merge` False)."""
        if not getattr(self, "deferred_attention_merge", True):
            return None
        a = self.args
        lib = _lib.load()
        splits = getattr(self, "attention_splits", None) or lib.ternaspmm_attention_partial_splits_kv(bsz, a.n_heads, a.n_kv_heads, max_seq)
        if splits < 1 or (splits == 1 and not single_split):
            return None
        # one buffer per batch size, kept while the model lives: a captured decode graph holds the raw pointer
        held = self.__dict__.setdefault("_attn_partial", {})
        if bsz not in held:
            nbytes = lib.ternaspmm_attention_partial_bytes(bsz, a.n_heads, a.head_dim)
            held[bsz] = torch.empty(nbytes // 4, dtype=torch.float32, device="cuda")
        return held[bsz], splits

    def attention_workspace(self, bsz: int):
        """Zero-filled scratch of the single-token attention (split over the cache); one per batch size, kept while
        the model lives (a captured decode graph holds the raw pointer)."""
        held = self.__dict__.setdefault("_attn_ws", {})
        if bsz not in held:
            a = self.args
            nbytes = _lib.load().ternaspmm_attention_workspace_bytes(bsz, a.n_heads, a.head_dim)
            held[bsz] = torch.zeros(nbytes, dtype=torch.int8, device="cuda")
        return held[bsz]

    def make_cache(self, bsz: int, max_seq: int):
        a = self.args
        shape = (bsz, a.n_kv_heads, max_seq, a.head_dim)
        dev = self.tok_embeddings.device
        return [(torch.zeros(shape, dtype=torch.bfloat16, device=dev), torch.zeros(shape, dtype=torch.bfloat16, device=dev))
                for _ in range(a.n_layers)]

    def forward(self, tokens: torch.Tensor, cache, pos_idx: torch.Tensor, trace=None, last_idx=None) -> torch.Tensor:
        """tokens int64 [B, T]; pos_idx int64 [T] = cache slots of the new tokens, the same for every sequence, or
        [B, T] = every sequence at its own slots (a batch of different prefix lengths).  Returns logits [B, vocab]
        of the last new token -- of new token last_idx[b] of sequence b when `last_idx` (int64 [B]) is given: the
        prompt pass of prompts padded to one length.  `trace`, if given, is called after every block as
        trace(index, stream_in, pending_in, stream_out, pending_out) (layer-by-layer checks against a golden)."""
        a = self.args
        bsz, t = tokens.shape
        max_seq = cache[0][0].shape[2]
        dev = tokens.device
        mask = None
        kernels_fit = self.layers[0].fused and a.head_dim in (64, 128) and max_seq <= 8192 and tokens.is_cuda
        one_launch_attention = kernels_fit and t == 1
        # one new token for a few sequences: the linears chained through producer-side norm statistics (forward_chain)
        chain = one_launch_attention and self.layers[0].act == "int8" and bsz <= max(self.chain_rows, self.split_rows) and getattr(self, "chain", True) and self.chain_supported()
        stats = None
        if chain and getattr(self, "step_inputs", True):
            # embedding rows, their partials under the first block's norm and the RoPE rows of the positions: one launch
            x, stats, cos, sin = step_inputs(tokens, pos_idx.reshape(-1), self.tok_embeddings, self.rope_tables(max_seq, dev), self.layers[0].attention_norm)
        else:
            rows = self.rope_tables(max_seq, dev).index_select(0, pos_idx.reshape(-1))   # fp32 [T | B*T, 2, head_dim / 2]
            cos, sin = rows[:, 0].contiguous(), rows[:, 1].contiguous()       # views when one row
            x = self.tok_embeddings[tokens.reshape(-1)]
        if kernels_fit and t > 1 and getattr(self, "kernel_prefill_attention", True):
            mask = KERNEL_ATTENTION
        elif not one_launch_attention:
            # causal over cache slots: new token at slot p sees slots <= p
            seen = torch.arange(max_seq, device=dev) <= pos_idx[..., None]    # [T | B, T][S]
            mask = seen[:, None] if pos_idx.dim() == 2 else seen[None, None]
        pending = None
        attn_ws = self.attention_workspace(bsz) if one_launch_attention else None     # layers run one after another: shared
        split = chain and bsz > self.chain_rows
        # split attention whose merge is left to its consumer: always for one sequence (the O projection's prologue merges);
        # for more only with long caches, where the shorter attention launch pays for the merge launch (8 sequences at slot
        # 1500: 1943 -> 1713 us per step; at slot 255 of 384 the pair of launches is 1.5 us slower than the unsplit one) --
        # (in the split chain that merge launch also norms and quantises the O projection's input; with short caches
        # the unsplit launch + the O projection with the norm inside stay ahead there too: 8 sequences, slot 255 of 384,
        # 1.198 against 1.218 ms per step -- `split_merge_quant` forces the split form)
        if one_launch_attention and self.layers[0].act == "int8" and (bsz == 1 or max_seq > (512 if split else self.defer_above)):
            attn_ws = self.attention_partial(bsz, max_seq) or attn_ws
        elif split and getattr(self, "split_merge_quant", False):
            attn_ws = self.attention_partial(bsz, max_seq, single_split=True) or attn_ws
        for index, (layer, (ck, cv)) in enumerate(zip(self.layers, cache)):
            x_in, pending_in = x, pending
            if chain:
                nxt = self.layers[index + 1].attention_norm if index + 1 < len(self.layers) else self.norm
                x, stats = layer.forward_chain(x, stats, ck, cv, pos_idx, cos, sin, attn_ws, nxt, split=split)
            else:
                x, pending = layer.forward(x, pending, ck, cv, pos_idx, cos, sin, mask, attn_ws)
            if trace is not None:
                trace(index, x_in, pending_in, x, pending)
        if last_idx is not None:                                              # padded prompts: each sequence's own last token
            pick = torch.arange(bsz, device=dev) * t + last_idx
            x, pending = x.index_select(0, pick), pending.index_select(0, pick)
        elif t > 1:                                                           # only the last new token feeds the head
            x, pending = x.view(bsz, t, a.dim)[:, -1].contiguous(), pending.view(bsz, t, a.dim)[:, -1].contiguous()
        if self.layers[0].fused and x.is_cuda:                                # last residual add + final norm: one launch
            x, _ = rmsnorm_quant(x, self.norm, a.norm_eps, residual=pending, quant=False)     # (chain: pending is None, the stream has it)
        else:
            x = rms_norm(x + pending, self.norm, a.norm_eps)
        if x.is_cuda and bsz <= 16 and a.dim % 32 == 0 and bsz * (2 * a.dim + 16) <= 160 * 1024:
            return lm_head(x, self.tok_embeddings)                            # tied LM head (model.py:367): one HBM-bound pass
        return F.linear(x, self.tok_embeddings)


@torch.inference_mode()
def greedy_decode(model: Transformer, prompt: torch.Tensor, gen_tokens: int, use_graph: bool = True, prompt_lens=None):
    """Prefill `prompt` [B, P], then `gen_tokens` greedy steps.  Returns (tokens [B, gen_tokens],
    prefill seconds, decode seconds).  The decode step (model forward + argmax + position bump) is
    captured once and replayed, so the host issues one graph launch per token.
    `prompt_lens` (int64 [B], each 1 .. P): the prompts have different lengths and are padded to P with any token
    (generate.py:244-262): sequence b's first generated token comes from its prompt token prompt_lens[b] - 1, and
    its n-th decode step runs at cache slot prompt_lens[b] + n -- every sequence at its own position."""
    bsz, plen = prompt.shape
    cache = model.make_cache(bsz, plen + gen_tokens)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    slots = torch.arange(plen, device="cuda")
    if prompt_lens is not None:
        return _greedy_decode_ragged(model, prompt, prompt_lens.to(device="cuda", dtype=torch.int64), gen_tokens, use_graph,
                                     cache, slots, ev)
    if use_graph:
        # the prompt pass as a graph too (generate.py:100-144): warm up on a side stream, capture, replay
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model.forward(prompt, cache, slots)
        torch.cuda.current_stream().wait_stream(side)
        prefill = torch.cuda.CUDAGraph()
        with torch.cuda.graph(prefill):
            logits = model.forward(prompt, cache, slots)
        torch.cuda.synchronize()
        ev[0].record()
        prefill.replay()
    else:
        ev[0].record()
        logits = model.forward(prompt, cache, slots)
    tok = argmax_rows(logits.contiguous())                                    # int64 [B, 1]
    ev[1].record()
    counters = torch.tensor([plen, 1], dtype=torch.int64, device="cuda")      # cache slot of the next token, tokens stored
    pos = counters[0:1]
    out = torch.empty((bsz, gen_tokens), dtype=torch.int64, device="cuda")
    out[:, 0:1] = tok
    state = greedy_step_state(bsz)

    def step():                                                               # the forward has read tok by the time it changes
        greedy_step(model.forward(tok, cache, pos), tok, out, counters, state)

    graph = None
    if use_graph:
        # warm up on a side stream (allocator, lazy inits), then restore the state and capture
        snap = (tok.clone(), counters.clone())
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        tok.copy_(snap[0]); counters.copy_(snap[1])
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        tok.copy_(snap[0]); counters.copy_(snap[1])
    torch.cuda.synchronize()
    ev[2].record()
    for _ in range(gen_tokens):
        if graph is not None:
            graph.replay()
        else:
            step()
    ev[3].record()
    torch.cuda.synchronize()
    return out, ev[0].elapsed_time(ev[1]) * 1e-3, ev[2].elapsed_time(ev[3]) * 1e-3


def _greedy_decode_ragged(model, prompt, prompt_lens, gen_tokens, use_graph, cache, slots, ev):
    """greedy_decode for prompts of different lengths: the prompt pass runs on the padded prompts (a padding token's
    cache rows are overwritten by the decode steps before any query can see them), the decode steps carry one cache
    position per sequence."""
    bsz = prompt.shape[0]
    ev[0].record()
    logits = model.forward(prompt, cache, slots, last_idx=prompt_lens - 1)
    tok = argmax_rows(logits.contiguous())                                    # int64 [B, 1]
    ev[1].record()
    seq_pos = prompt_lens.clone().view(bsz, 1)                                # cache slot of every sequence's next token
    counters = torch.tensor([0, 1], dtype=torch.int64, device="cuda")         # [1]: tokens stored in the history
    out = torch.empty((bsz, gen_tokens), dtype=torch.int64, device="cuda")
    out[:, 0:1] = tok
    state = greedy_step_state(bsz)

    def step():
        greedy_step(model.forward(tok, cache, seq_pos), tok, out, counters, state)
        seq_pos.add_(1)

    graph = None
    if use_graph:
        snap = (tok.clone(), counters.clone(), seq_pos.clone())
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        tok.copy_(snap[0]); counters.copy_(snap[1]); seq_pos.copy_(snap[2])
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        tok.copy_(snap[0]); counters.copy_(snap[1]); seq_pos.copy_(snap[2])
    torch.cuda.synchronize()
    ev[2].record()
    for _ in range(gen_tokens):
        if graph is not None:
            graph.replay()
        else:
            step()
    ev[3].record()
    torch.cuda.synchronize()
    return out, ev[0].elapsed_time(ev[1]) * 1e-3, ev[2].elapsed_time(ev[3]) * 1e-3
