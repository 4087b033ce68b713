"""The end-to-end configuration at FULL size: BitNet-b1.58-2B shape (30 layers, hidden 2560, 20 / 5 heads of
128, FFN 6912, vocabulary 128256), ternary P(0) = 0.40, batch 1 and 8, 128-token prompt.

Layer by layer with teacher forcing: every block's GPU input (residual stream + the pending FFN output) is fed
to a CPU twin of that ONE block, written here from the reference's block structure (model.py:196-335: fused
wqkv -> RoPE on adjacent pairs -> cache -> attention -> attn_sub_norm -> wo; residual; ffn_norm -> w13 ->
relu(x1)^2 * x3 -> ffn_sub_norm -> w2; SpBitLinear.quant_input in front of every linear, model.py:120-133) with
dense fp32 matmuls on the ORIGINAL ternary matrices -- the GPU side gets them through the host encoder, the
load-time repack and the kernels.  The blocks record the int8 activations and scales every linear consumed
(`Block.capture`), and the twin's linears run on exactly those: every one of the 120 linears of a pass is therefore
compared BIT FOR BIT at full size, and so are the residual stream, the gate and the v rows of the cache; only the
norms (one bf16 step: a parallel fp32 sum of squares), the rotation (one step) and the attention (2^-7 of a head's
largest output) keep a tolerance, each checked where it arises.  A wrong kernel shows up in the layer and pass where
it ran.  Passes: the 128-token prompt (large-M
kernels, multi-token attention) and two single-token steps (prologue-inside small-M kernels at K = 2560 and
K = 6912, RoPE + cache write + attention in one launch over head_dim 128, the second step with the prefetching
variant), then the final norm and the 128256-wide LM head.  Plus: a captured decode graph gives the tokens of
eager execution at full size.
"""

import numpy as np
import pytest
import torch

from oracle import terna_oracle as O

pytestmark = pytest.mark.gpu

PROMPT = 128
STEPS = 2


def ternary_host(n, k, gen):
    """iid ternary int8 [n, k] on the host: P(0) = 0.4, P(+1) = P(-1) = 0.3.  Drawn with the generator's device
    (the GPU draws 70 M values in no time; the matrix then lives on the host as the twin's dense weight and goes
    to the GPU path only through the host encoder)."""
    r = torch.randint(0, 10, (n, k), generator=gen, dtype=torch.int8, device=gen.device)
    return ((r >= 4).to(torch.int8) - 2 * (r >= 7).to(torch.int8)).cpu()


def upload_linear(w, scales, act="int8"):
    """Dense ternary matrix -> reference format (host encoder) -> device -> P2 (load-time repack) -> TernaryLinear."""
    import ternainfer_amd as T
    from ternainfer_amd.model import TernaryLinear
    n, k = w.shape
    vals, off, med, bm = T.compress_weight(w)
    packed = T.repack_weight(vals.cuda(), off.cuda(), med.cuda(), bm.cuda(), n, k)
    torch.cuda.synchronize()
    ws = torch.zeros(4, dtype=torch.bfloat16)
    ws[:len(scales)] = torch.tensor(scales, dtype=torch.bfloat16)
    return TernaryLinear(k, n, packed, ws.cuda(), act)


def build_model(args, seed):
    """Transformer with every ternary matrix drawn on the host; returns (model, per-layer host matrices)."""
    from ternainfer_amd.model import Block, Transformer
    gen = torch.Generator().manual_seed(seed)
    wgen = torch.Generator(device="cuda").manual_seed(seed + 1)
    model = Transformer.__new__(Transformer)
    model.args = args
    model.tok_embeddings = (torch.randn((args.vocab_size, args.dim), generator=gen) * 0.02).to(torch.bfloat16).cuda()
    model.norm = (1 + 0.1 * torch.randn(args.dim, generator=gen)).to(torch.bfloat16).cuda()
    d, hd, f = args.dim, args.head_dim, args.ffn_dim
    qkv_n = (args.n_heads + 2 * args.n_kv_heads) * hd
    model.layers, host = [], []
    for _ in range(args.n_layers):
        blk = Block(args, None, "int8")
        sc = lambda n: torch.empty(n).uniform_(0.5, 2.0, generator=gen).to(torch.bfloat16).float().tolist()
        mats = {"wqkv": (ternary_host(qkv_n, d, wgen), sc(3)), "wo": (ternary_host(d, d, wgen), sc(1)),
                "w13": (ternary_host(2 * f, d, wgen), sc(2)), "w2": (ternary_host(d, f, wgen), sc(1))}
        norms = {nm: (1 + 0.1 * torch.randn(width, generator=gen)).to(torch.bfloat16)
                 for nm, width in (("attention_norm", d), ("attn_sub_norm", d), ("ffn_norm", d), ("ffn_sub_norm", f))}
        for nm, (w, s) in mats.items():
            setattr(blk, nm, upload_linear(w, s))
        for nm, v in norms.items():
            setattr(blk, nm, v.cuda())
        model.layers.append(blk)
        host.append((mats, norms))
    return model, host


# ---------------------------------------------------------------------------------------------- CPU twin of one block
def cpu_rms(h, w, eps):
    hf = h.double()
    return (hf * torch.rsqrt(hf.pow(2).mean(-1, keepdim=True) + eps) * w.double()).to(torch.bfloat16)


def cpu_quant(y):
    """quant_input as the library defines it by default: fp32 product, bf16-rounded s in the product."""
    yf = y.float()
    s = (127.0 / yf.abs().amax(-1, keepdim=True).clamp_(min=1e-5)).to(torch.bfloat16)
    return (yf * s.float()).round().clamp(-128, 127).to(torch.int8), s.reshape(-1)


def cpu_matmul_epilogue(xq, s, w_f32, scales, n):
    """Exact integer matmul on given int8 activations + the library's epilogue rule by M: (acc / s) * ws[g] up to 64
    rows, acc * (ws[g] / s) with g per 128-column tile above.  Every operation is one IEEE fp32 operation."""
    m = xq.shape[0]
    acc = xq.float() @ w_f32.T                          # integers below 2^24: exact in fp32
    sf = s.float().reshape(m, 1)
    ws = torch.tensor(scales, dtype=torch.float32)
    cols = np.arange(n)
    if m <= 64:
        g = torch.from_numpy(O.ws_group_decode(cols, n, len(scales)))
        return ((acc / sf) * ws[g]).to(torch.bfloat16)
    g = torch.from_numpy(O.ws_group_prefill(cols, n, len(scales)))
    return (acc * (ws[g][None, :] / sf)).to(torch.bfloat16)


def cpu_rope_adjacent(x, cos, sin):
    """x [B, T, heads, D] bf16; cos / sin [T, D/2]; pairs (2j, 2j+1)."""
    xf = x.float()
    x1, x2 = xf[..., 0::2], xf[..., 1::2]
    c, s = cos[None, :, None, :], sin[None, :, None, :]
    return torch.stack([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1).flatten(-2).to(torch.bfloat16)


def bf16_steps(a, b):
    """Distance in bf16 steps (monotone integer image of the storage)."""
    def key(t):
        v = t.contiguous().view(torch.int16).to(torch.int32)
        return torch.where(v < 0, -(v & 0x7FFF), v)
    return (key(a) - key(b)).abs()


class Worst:
    def __init__(self):
        self.v = {}

    def note(self, name, value):
        self.v[name] = max(self.v.get(name, 0.0), float(value))


def check_quantiser(tag, y_twin, xq, s, worst, max_step, max_frac):
    """The GPU's (xq, s) against the quantisation of the twin's float64 norm output: the scale within one bf16 step (or
    the scale of a row maximum one bf16 step beside the twin's);
    on rows whose scale agrees the integers within `max_step`, differing on at most `max_frac` of the elements.
    Observed worst over the batch sizes, 30 layers and 3 passes: one step on 5e-5 of the elements where the norm's
    input is known exactly (bound 2e-3), on 8e-4 behind the attention that is merged inside the O projection, where
    the twin's input comes from its own float64 attention (bound 1e-2)."""
    q_t, s_t = cpu_quant(y_twin)
    ds = bf16_steps(s, s_t)
    # The fp32 norm may round a row's largest element to the bf16 neighbour of the float64 norm's; where that value's
    # mantissa is near 1 and the scale's near 2, one step of the maximum is two steps of 127 / maximum.  So a scale more
    # than one step off must be the exact scale of a maximum one bf16 step beside the twin's.
    top = y_twin.float().abs().amax(-1).to(torch.bfloat16).view(torch.int16).to(torch.int32)
    beside = [(127.0 / (top + d).to(torch.int16).view(torch.bfloat16).float().clamp(min=1e-5)).to(torch.bfloat16) for d in (-1, 1)]
    ok = (ds <= 1) | (s == beside[0]) | (s == beside[1])
    assert bool(ok.all()), f"{tag}: activation scale {int(ds[~ok].max())} bf16 steps off"
    same = ds == 0
    assert bool(same.any()), f"{tag}: no row with an agreeing scale"
    dq = (xq[same].to(torch.int32) - q_t[same].to(torch.int32)).abs()
    frac = (dq != 0).float().mean().item()
    assert int(dq.max()) <= max_step and frac <= max_frac, f"{tag}: int8 activations differ by up to {int(dq.max())} on {frac:.4f}"
    worst.note(tag.split()[-1] + " dq max", dq.max())
    worst.note(tag.split()[-1] + " dq frac", frac)


def cpu_block_check(args, mats, norms, rec, x_in, pend_in, x_out, pend_out, cache_before, cache_after, pos, rope, tag, worst):
    """One block of one pass.  `rec`: what the block recorded, in order -- ("wqkv" | "wo" | "w13" | "w2", xq, s, the
    linear's own output) and ("attention", the attention output) where one exists in memory.
      * every linear: its output must be the exact integer matmul + epilogue of the (xq, s) IT consumed -- bit for bit,
        all columns, at full size;
      * every norm + quantisation: (xq, s) against the float64 norm of an input whose bits are known exactly;
      * residual stream, gate, RoPE'd cache rows: exact bf16 arithmetic on those outputs;
      * attention: within 2^-7 of the head's largest output where it is in memory, else through the O projection's xq."""
    a = args
    bsz = cache_before[0].shape[0]
    t = len(pos)
    hd, nh, nkv = a.head_dim, a.n_heads, a.n_kv_heads
    lin = {name: (xq, s, out) for name, xq, s, out in rec if name != "attention"}
    attn_out = next((out for name, _, _, out in rec if name == "attention"), None)
    chain = pend_out is None                                            # the decode steps: the stream already holds the FFN output

    def linear(name, n):
        xq, s, out = lin[name]
        want = cpu_matmul_epilogue(xq, s, mats[name][0], mats[name][1], n)
        assert torch.equal(out, want), f"{tag} {name}: output is not the integer matmul + epilogue of its own (xq, s)"
        return out

    h0 = x_in if pend_in is None else x_in + pend_in                    # bf16 + bf16 -> bf16: the stream this block reads
    check_quantiser(f"{tag} wqkv", cpu_rms(h0, norms["attention_norm"], a.norm_eps), lin["wqkv"][0], lin["wqkv"][1], worst, 1, 0.002)
    qkv = linear("wqkv", (nh + 2 * nkv) * hd).view(bsz, t, nh + 2 * nkv, hd)
    cos, sin = rope[pos, 0], rope[pos, 1]                               # the fp32 table rows the kernels were handed
    q = cpu_rope_adjacent(qkv[:, :, :nh], cos, sin)
    k = cpu_rope_adjacent(qkv[:, :, nh:nh + nkv], cos, sin)
    v = qkv[:, :, nh + nkv:]
    # the new cache rows: v is a copy; k went through the rotation, whose fp32 products and sums are each rounded once
    # (no fused multiply-add on either side): the same bits
    assert torch.equal(cache_after[1][:, :, pos], v.transpose(1, 2)), f"{tag}: v rows"
    assert torch.equal(cache_after[0][:, :, pos], k.transpose(1, 2)), f"{tag}: k rows"
    ck, cv = cache_before[0].clone(), cache_before[1].clone()
    ck[:, :, pos] = cache_after[0][:, :, pos]                           # the GPU's own rows: errors do not compound
    cv[:, :, pos] = cache_after[1][:, :, pos]
    rep = nh // nkv
    last = pos[-1] + 1
    kk = ck[:, :, :last].double().repeat_interleave(rep, dim=1)         # [B, H, last, D]
    vv = cv[:, :, :last].double().repeat_interleave(rep, dim=1)
    sc = torch.einsum("bthd,bhsd->bhts", q.double(), kk) * hd ** -0.5
    visible = torch.arange(last)[None, :] <= torch.tensor(pos)[:, None] # [T, last]: slot p sees slots <= p
    sc = sc.masked_fill(~visible[None, None], float("-inf"))
    o64 = torch.einsum("bhts,bhsd->bthd", torch.softmax(sc, dim=-1), vv)           # [B, T, H, D]
    o_twin = o64.to(torch.bfloat16).reshape(bsz * t, nh * hd)
    if attn_out is not None:
        err = (attn_out.double().view(bsz, t, nh, hd) - o64).abs().amax(dim=-1)
        bound = o64.abs().amax(dim=-1) * 2.0 ** -7 + 1e-30
        assert bool((err <= bound).all()), f"{tag}: attention output beyond 2^-7 of the head's largest value"
        worst.note("attention err / head max", (err / bound).max() * 2.0 ** -7)
        o_in = attn_out
        check_quantiser(f"{tag} wo", cpu_rms(o_in, norms["attn_sub_norm"], a.norm_eps), lin["wo"][0], lin["wo"][1], worst, 1, 0.002)
    else:   # merged inside the O projection's prologue: only its quantised form exists
        check_quantiser(f"{tag} wo", cpu_rms(o_twin, norms["attn_sub_norm"], a.norm_eps), lin["wo"][0], lin["wo"][1], worst, 1, 0.01)
    attn = linear("wo", a.dim)
    h = h0 + attn
    check_quantiser(f"{tag} w13", cpu_rms(h, norms["ffn_norm"], a.norm_eps), lin["w13"][0], lin["w13"][1], worst, 1, 0.002)
    if chain:
        # gate+up leaves relu(x1)^2 * x3 directly: the twin forms x13 from the same (xq, s) and applies the gate
        xq, s, inner = lin["w13"]
        x13 = cpu_matmul_epilogue(xq, s, mats["w13"][0], mats["w13"][1], 2 * a.ffn_dim)
        x1, x3 = x13.chunk(2, dim=-1)
        want = (torch.relu(x1) ** 2) * x3
        assert torch.equal(inner, want), f"{tag} w13: gate output is not relu(x1)^2 * x3 of the exact x13"
    else:
        x1, x3 = linear("w13", 2 * a.ffn_dim).chunk(2, dim=-1)
        inner = (torch.relu(x1) ** 2) * x3
    check_quantiser(f"{tag} w2", cpu_rms(inner, norms["ffn_sub_norm"], a.norm_eps), lin["w2"][0], lin["w2"][1], worst, 1, 0.002)
    ffn = linear("w2", a.dim)
    if chain:
        assert torch.equal(x_out, h + ffn), f"{tag}: stream after the block"
    else:
        assert torch.equal(x_out, h) and torch.equal(pend_out, ffn), f"{tag}: stream / pending FFN output"


def close(got, want, what, rel, rms):
    """max|err| <= rel * max|ref| and rms(err) <= rms * rms(ref).  Returns the two ratios."""
    got, want = got.double(), want.double()
    err, ref = (got - want).abs().max().item(), want.abs().max().item()
    r = ((got - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt().clamp_(min=1e-30)).item()
    assert err <= rel * ref and r <= rms, f"{what}: max err {err:.4g} vs max|ref| {ref:.4g}, relative rms error {r:.3g}"
    return err / ref, r


@pytest.fixture(scope="module")
def full_model():
    from ternainfer_amd.model import ModelArgs
    args = ModelArgs()
    assert (args.dim, args.n_layers, args.n_heads, args.n_kv_heads, args.vocab_size, args.ffn_dim, args.head_dim) == \
        (2560, 30, 20, 5, 128256, 6912, 128)
    print("[case] building the 2B-shaped model (host matrices -> encoder -> repack)", flush=True)
    return (args,) + build_model(args, seed=20260500)


@pytest.mark.parametrize("bsz", [1, 8, 12, 16])
def test_full_size_blocks_match_cpu_twin_layer_by_layer(full_model, bsz):
    args, model, host = full_model
    gen = torch.Generator().manual_seed(20260500 + bsz)
    prompt = torch.randint(0, args.vocab_size, (bsz, PROMPT), generator=gen).cuda()
    max_seq = PROMPT + STEPS
    cache = model.make_cache(bsz, max_seq)
    passes = []                                       # (slots, per-layer records, cache snapshot BEFORE the pass, logits)
    cpu = lambda t: None if t is None else t.cpu()

    def run(tokens, slots):
        before = [(ck.cpu(), cv.cpu()) for ck, cv in cache]
        rec = []
        for blk in model.layers:
            blk.capture = []
        logits = model.forward(tokens, cache, torch.tensor(slots, device="cuda"),
                               trace=lambda i, xi, pi, xo, po: rec.append((cpu(xi), cpu(pi), cpu(xo), cpu(po))))
        torch.cuda.synchronize()
        caps = [[(nm, cpu(xq), cpu(s), cpu(out)) for nm, xq, s, out in blk.capture] for blk in model.layers]
        for blk in model.layers:
            blk.capture = None
        after = [(ck.cpu(), cv.cpu()) for ck, cv in cache]
        passes.append((slots, rec, caps, before, after, logits.cpu()))
        return logits

    with torch.inference_mode():
        print(f"[case] full-size model batch {bsz}: prompt pass", flush=True)
        logits = run(prompt, list(range(PROMPT)))
        for step in range(STEPS):
            tok = logits.float().argmax(dim=-1, keepdim=True)
            model.enable_prefetch(step == 1)          # the second step through the prefetching attention launch
            print(f"[case] full-size model batch {bsz}: single-token step {step}", flush=True)
            logits = run(tok, [PROMPT + step])
        model.enable_prefetch(False)

        worst = Worst()
        rope = model.rope_tables(max_seq, prompt.device).cpu()        # fp32 [max_seq, 2, head_dim / 2]: cos rows, sin rows
        for layer, (mats, norms) in enumerate(host):
            dense = {nm: (w.float(), s) for nm, (w, s) in mats.items()}          # ~280 MB, released per layer
            for pi, (slots, rec, caps, before, after, _) in enumerate(passes):
                xi, pend, xo, po = rec[layer]
                names = [c[0] for c in caps[layer]]
                assert [n for n in names if n != "attention"] == ["wqkv", "wo", "w13", "w2"], names
                cpu_block_check(args, dense, norms, caps[layer], xi, pend, xo, po, before[layer], after[layer], slots, rope,
                                f"batch {bsz} layer {layer} pass {pi}", worst)
            del dense
        print(f"[info] batch {bsz}: worst over 30 layers x 3 passes: " + ", ".join(f"{k} {v:.3g}" for k, v in sorted(worst.v.items())),
              flush=True)

        # final residual add + norm + tied bf16 LM head (model.py:367, 449-455) on the last block's GPU outputs
        emb = model.tok_embeddings.cpu().float()
        for pi, (slots, rec, _, _, _, got_logits) in enumerate(passes):
            _, _, xo, po = rec[-1]
            t = len(slots)
            x_last = xo.view(bsz, t, args.dim)[:, -1]
            if po is not None:
                x_last = x_last + po.view(bsz, t, args.dim)[:, -1]
            y = cpu_rms(x_last, model.norm.cpu(), args.norm_eps)
            want = (y.float() @ emb.T)
            r = close(got_logits, want, f"batch {bsz} pass {pi} logits", 1e-2, 4e-3)
            print(f"[info] batch {bsz} pass {pi} logits: {r}", flush=True)


@pytest.mark.parametrize("bsz", [1, 8, 12, 16])
def test_full_size_decode_graph_gives_the_tokens_of_eager_execution(full_model, bsz):
    from ternainfer_amd.model import greedy_decode
    args, model, _ = full_model
    prompt = torch.randint(0, args.vocab_size, (bsz, PROMPT), generator=torch.Generator().manual_seed(20260510 + bsz)).cuda()
    model.enable_prefetch(True, ("wo", "w13", "w2", "next_wqkv", "norms") if bsz == 1 else ("wo", "w13"))
    print(f"[case] full-size greedy decode batch {bsz}: graph vs eager, 16 tokens", flush=True)
    a, _, _ = greedy_decode(model, prompt, 16, use_graph=True)
    b, _, _ = greedy_decode(model, prompt, 16, use_graph=False)
    model.enable_prefetch(False)
    assert torch.equal(a, b)
    assert int(a.min()) >= 0 and int(a.max()) < args.vocab_size
