"""The 2B-shaped harness at toy size: logits through libternaspmm.so against a CPU golden that
runs the SAME forward with dense fp64 ternary matmuls (weights unpacked from the P2 buffers)."""
import numpy as np
import pytest
import torch

from oracle import terna_oracle as O

pytestmark = pytest.mark.gpu


class DenseLinearCPU:
    """CPU stand-in for TernaryLinear: same activation quantisation, integer matmul in fp64,
    the decode-path epilogue (acc / s) * ws[g] with the reference's group rule."""

    def __init__(self, lin, act, w=None):
        """`w`: the dense ternary matrix if the caller has it from elsewhere; else unpacked from lin.packed."""
        self.n, self.k, self.act = lin.n, lin.k, act
        if w is None:
            packed = lin.packed.cpu().numpy().view(np.uint32)
            w = O.unpack_p2(packed, lin.n, lin.k)
        self.w = torch.from_numpy(np.asarray(w).astype(np.float64))
        groups = O.ws_group_decode(np.arange(lin.n), lin.n, lin.ws_num)
        self.ws = lin.ws.float().cpu().double()[torch.from_numpy(groups)]

    def __call__(self, x):
        if self.act == "int8":
            xf = x.float()
            s = (127 / xf.abs().amax(dim=-1, keepdim=True).clamp_(min=1e-5)).to(torch.bfloat16)
            xq = (xf * s.float()).round().clamp(-128, 127)
            acc = xq.double() @ self.w.T
            return ((acc / s.double()) * self.ws).to(torch.bfloat16)
        return ((x.double() @ self.w.T) * self.ws).to(torch.bfloat16)


@pytest.mark.parametrize("act", ["int8", "bf16"])
def test_toy_model_matches_cpu_golden(act):
    import copy
    from ternainfer_amd.model import ModelArgs, Transformer
    args = ModelArgs(dim=256, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=1024, ffn_dim=384)
    model = Transformer(args, seed=7, act=act)
    tokens = torch.randint(0, args.vocab_size, (2, 24), generator=torch.Generator().manual_seed(8))
    print(f"[case] toy model forward act={act}", flush=True)
    with torch.inference_mode():
        got = model.forward(tokens.cuda(), model.make_cache(2, 32), torch.arange(24, device="cuda")).float().cpu()

        twin = copy.copy(model)
        twin.tok_embeddings = model.tok_embeddings.cpu()
        twin.norm = model.norm.cpu()
        twin.layers = []
        for blk in model.layers:
            b = copy.copy(blk)
            b.fused = False                      # the CPU twin runs the same block with plain torch ops
            for name in ("wqkv", "wo", "w13", "w2"):
                setattr(b, name, DenseLinearCPU(getattr(blk, name), act))
            for name in ("attention_norm", "ffn_norm", "attn_sub_norm", "ffn_sub_norm"):
                setattr(b, name, getattr(blk, name).cpu())
            twin.layers.append(b)
        want = twin.forward(tokens, twin.make_cache(2, 32), torch.arange(24)).float()
    err = (got - want).abs().max().item()
    ref = want.abs().max().item()
    assert err <= 3e-2 * ref, (err, ref)
    assert torch.nn.functional.cosine_similarity(got.flatten(), want.flatten(), dim=0).item() > 0.999


def test_toy_model_fused_prologue_equals_torch_ops():
    """Same model, norms / gate / quantisation through the fused kernels vs through torch ops."""
    from ternainfer_amd.model import ModelArgs, Transformer
    args = ModelArgs(dim=256, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=1024, ffn_dim=384)
    tokens = torch.randint(0, args.vocab_size, (2, 24), generator=torch.Generator().manual_seed(11)).cuda()
    outs = []
    model = Transformer(args, seed=12, act="int8")
    for fused in (True, False):
        for blk in model.layers:
            blk.fused = fused
        with torch.inference_mode():
            outs.append(model.forward(tokens, model.make_cache(2, 32), torch.arange(24, device="cuda")).float())
    err = (outs[0] - outs[1]).abs().max().item()
    assert err <= 3e-2 * outs[1].abs().max().item()
    assert torch.nn.functional.cosine_similarity(outs[0].flatten(), outs[1].flatten(), dim=0).item() > 0.999


def test_toy_model_greedy_decode_graph_equals_eager():
    from ternainfer_amd.model import ModelArgs, Transformer, greedy_decode
    args = ModelArgs(dim=256, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=1024, ffn_dim=384)
    model = Transformer(args, seed=9, act="int8")
    prompt = torch.randint(0, args.vocab_size, (2, 16), generator=torch.Generator().manual_seed(10)).cuda()
    print("[case] toy model greedy decode, graph vs eager", flush=True)
    a, _, _ = greedy_decode(model, prompt, 12, use_graph=True)
    b, _, _ = greedy_decode(model, prompt, 12, use_graph=False)
    assert torch.equal(a, b)
    model.enable_prefetch()                      # idle CUs of the attention launch prefetch the next weights: same tokens
    c, _, _ = greedy_decode(model, prompt, 12, use_graph=True)
    model.enable_prefetch(False)
    assert torch.equal(a, c)


@pytest.mark.parametrize("bsz,plen,slots", [(3, 20, 40), (6, 20, 40), (12, 20, 40), (16, 20, 40), (6, 560, 600), (12, 1040, 1100), (2, 700, 720)])
def test_toy_model_decode_step_forms_agree(bsz, plen, slots):
    """One-token steps of several sequences: the chained forms (up to four sequences the statistics are consumed inside the
    next linear, above by the element-wise quantise launch; from nine on the O projection takes the norm kernel's rows)
    against the step of plain launches; greedy tokens of the replayed graph against eager execution.  With the longer caches
    the chained steps split their attention (one workgroup per kv head) and leave the merge to the launch that also norms
    and quantises the O projection's input."""
    from ternainfer_amd.model import ModelArgs, Transformer, greedy_decode
    args = ModelArgs(dim=256, n_layers=3, n_heads=4, n_kv_heads=2, vocab_size=1024, ffn_dim=384)
    model = Transformer(args, seed=61, act="int8")
    assert model.chain_supported()
    prompt = torch.randint(0, args.vocab_size, (bsz, plen), generator=torch.Generator().manual_seed(62 + bsz)).cuda()
    print(f"[case] toy model, {bsz} sequences, {slots} cache slots: chained decode step against plain launches", flush=True)
    outs = []
    with torch.inference_mode():
        for chain in (True, False):
            model.chain = chain
            cache = model.make_cache(bsz, slots)
            model.forward(prompt, cache, torch.arange(plen, device="cuda"))
            outs.append(model.forward(prompt[:, -1:].contiguous(), cache, torch.tensor([plen], device="cuda")).float())
    model.chain = True
    if slots > 512 and bsz > 1:
        assert model.attention_partial(bsz, slots) is not None             # the split attention is the path that ran
    assert outs[0].shape == (bsz, args.vocab_size)
    err = (outs[0] - outs[1]).abs().max().item()
    assert err <= 3e-2 * outs[1].abs().max().item(), err
    assert torch.nn.functional.cosine_similarity(outs[0].flatten(), outs[1].flatten(), dim=0).item() > 0.9995
    gen = min(10, slots - plen)
    a, _, _ = greedy_decode(model, prompt, gen, use_graph=True)
    b, _, _ = greedy_decode(model, prompt, gen, use_graph=False)
    assert torch.equal(a, b)


@pytest.mark.parametrize("head_dim,prefetch", [(64, False), (128, True)])
def test_toy_model_prompts_of_different_lengths_in_one_batch(head_dim, prefetch):
    """Three prompts of different lengths, padded to one length and decoded together with every sequence at its own
    cache position (generate.py:244-305 hands its attention one kv_seqlen per sequence), against each prompt decoded
    alone: the same tokens, eager and as a replayed graph; and against the forward without the fused kernels (torch
    RoPE, per-sequence masks, SDPA) on the first decode step."""
    from ternainfer_amd.model import ModelArgs, Transformer, greedy_decode
    args = ModelArgs(dim=4 * head_dim, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=1024, ffn_dim=384)
    model = Transformer(args, seed=31, act="int8")
    model.enable_prefetch(prefetch)
    lens = [5, 12, 9]
    gen = torch.Generator().manual_seed(32)
    prompts = [torch.randint(0, args.vocab_size, (1, n), generator=gen).cuda() for n in lens]
    padded = torch.full((3, max(lens)), 7, dtype=torch.int64, device="cuda")
    for i, p in enumerate(prompts):
        padded[i, :lens[i]] = p[0]
    print(f"[case] toy model, ragged batch head_dim={head_dim} prefetch={prefetch}", flush=True)
    alone = torch.cat([greedy_decode(model, p, 8, use_graph=False)[0] for p in prompts])
    together, _, _ = greedy_decode(model, padded, 8, use_graph=False, prompt_lens=torch.tensor(lens))
    assert torch.equal(alone, together)
    replayed, _, _ = greedy_decode(model, padded, 8, use_graph=True, prompt_lens=torch.tensor(lens))
    assert torch.equal(alone, replayed)
    # one decode step with per-sequence positions: fused kernels against torch ops
    with torch.inference_mode():
        outs = []
        for fused in (True, False):
            for blk in model.layers:
                blk.fused = fused
            cache = model.make_cache(3, 24)
            model.forward(padded, cache, torch.arange(max(lens), device="cuda"))
            seq_pos = torch.tensor(lens, device="cuda").view(3, 1)
            outs.append(model.forward(together[:, :1].contiguous(), cache, seq_pos).float())
        for blk in model.layers:
            blk.fused = True
    err = (outs[0] - outs[1]).abs().max().item()
    assert err <= 3e-2 * outs[1].abs().max().item()
    assert torch.nn.functional.cosine_similarity(outs[0].flatten(), outs[1].flatten(), dim=0).item() > 0.999


@pytest.mark.parametrize("head_dim,splits", [(64, 2), (128, 4), (128, 8)])
def test_toy_model_attention_merge_deferred_to_the_o_projection(head_dim, splits):
    """One sequence: the decode step whose attention leaves the merge of its splits to the O projection's prologue
    against the step with the attention in one piece -- logits within the tolerance of the two summation orders,
    the greedy tokens of a replayed graph equal to eager execution."""
    from ternainfer_amd.model import ModelArgs, Transformer, greedy_decode
    args = ModelArgs(dim=4 * head_dim, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=1024, ffn_dim=384)
    model = Transformer(args, seed=41, act="int8")
    prompt = torch.randint(0, args.vocab_size, (1, 150), generator=torch.Generator().manual_seed(42)).cuda()
    print(f"[case] toy model, deferred attention merge head_dim={head_dim} splits={splits}", flush=True)
    outs = []
    with torch.inference_mode():
        for deferred in (True, False):
            model.deferred_attention_merge = deferred
            model.attention_splits = splits
            cache = model.make_cache(1, 200)
            model.forward(prompt, cache, torch.arange(150, device="cuda"))
            outs.append(model.forward(prompt[:, -1:].contiguous(), cache, torch.tensor([150], device="cuda")).float())
    err = (outs[0] - outs[1]).abs().max().item()
    assert err <= 3e-2 * outs[1].abs().max().item(), err
    assert torch.nn.functional.cosine_similarity(outs[0].flatten(), outs[1].flatten(), dim=0).item() > 0.9995
    model.deferred_attention_merge = True
    a, _, _ = greedy_decode(model, prompt, 10, use_graph=True)
    b, _, _ = greedy_decode(model, prompt, 10, use_graph=False)
    assert torch.equal(a, b)
    model.enable_prefetch()
    c, _, _ = greedy_decode(model, prompt, 10, use_graph=True)
    assert torch.equal(a, c)


def test_toy_model_several_sequences_long_cache_deferred_merge():
    """Several sequences with a cache of more than 1024 slots: the harness splits the single-token attention and leaves
    the merge to a launch of its own in front of the O projection (ternaspmm_attention_merge).  Logits against the step
    with the attention in one piece; greedy tokens of a replayed graph against eager execution; every row of the batch
    must come out (the O projection sees one row per sequence)."""
    from ternainfer_amd.model import ModelArgs, Transformer, greedy_decode
    args = ModelArgs(dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=1024, ffn_dim=384)
    model = Transformer(args, seed=43, act="int8")
    bsz, plen, cache_slots = 3, 1040, 1100
    prompt = torch.randint(0, args.vocab_size, (bsz, plen), generator=torch.Generator().manual_seed(44)).cuda()
    print("[case] toy model, 3 sequences, 1100-slot cache, deferred attention merge", flush=True)
    assert model.attention_partial(bsz, cache_slots) is not None          # the path under test is the one that runs
    outs = []
    with torch.inference_mode():
        for deferred in (True, False):
            model.deferred_attention_merge = deferred
            cache = model.make_cache(bsz, cache_slots)
            model.forward(prompt, cache, torch.arange(plen, device="cuda"))
            outs.append(model.forward(prompt[:, -1:].contiguous(), cache, torch.tensor([plen], device="cuda")).float())
    assert outs[0].shape == outs[1].shape and outs[0].shape[0] == bsz
    err = (outs[0] - outs[1]).abs().max().item()
    assert err <= 3e-2 * outs[1].abs().max().item(), err
    assert torch.nn.functional.cosine_similarity(outs[0].flatten(), outs[1].flatten(), dim=0).item() > 0.9995
    model.deferred_attention_merge = True
    a, _, _ = greedy_decode(model, prompt, 70, use_graph=True)            # plen + 70 > 1024 slots
    b, _, _ = greedy_decode(model, prompt, 70, use_graph=False)
    assert torch.equal(a, b)


def test_toy_model_prompt_pass_kernel_attention_sdpa_and_graph_replays():
    """The prompt pass through the library's multi-token attention against the same pass through PyTorch's SDPA, and
    the captured prompt graph against eager execution on several replays with eager work and synchronisations between
    them (a captured node that misbehaves from the second replay on would show here)."""
    from ternainfer_amd.model import ModelArgs, Transformer
    args = ModelArgs(dim=256, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=1024, ffn_dim=384)
    model = Transformer(args, seed=13, act="int8")
    tokens = torch.randint(0, args.vocab_size, (2, 40), generator=torch.Generator().manual_seed(14)).cuda()
    slots = torch.arange(40, device="cuda")
    print("[case] toy model prompt pass: kernel attention vs SDPA, graph replays", flush=True)
    with torch.inference_mode():
        eager = model.forward(tokens, model.make_cache(2, 48), slots).float()
        model.kernel_prefill_attention = False
        sdpa = model.forward(tokens, model.make_cache(2, 48), slots).float()
        model.kernel_prefill_attention = True
        assert (eager - sdpa).abs().max().item() <= 3e-2 * sdpa.abs().max().item()
        assert torch.nn.functional.cosine_similarity(eager.flatten(), sdpa.flatten(), dim=0).item() > 0.999
        cache = model.make_cache(2, 48)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model.forward(tokens, cache, slots)
        torch.cuda.current_stream().wait_stream(side)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            captured = model.forward(tokens, cache, slots)
        for _ in range(3):
            captured.zero_()
            for ck, cv in cache:
                ck.zero_(); cv.zero_()
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(captured.float(), eager)


def test_converted_checkpoint_loads_and_matches_cpu_golden(tmp_path):
    """fp32 state dict -> converter -> three files -> Transformer.from_checkpoint; the CPU golden is built
    from the converter's int8 matrices (not from the packed buffers), so the loader and the repack are
    inside the comparison."""
    import copy
    import ternainfer_amd as T
    from ternainfer_amd.model import ModelArgs, Transformer
    from tests.test_checkpoint_convert import toy_state
    cfg = T.CheckpointShape(dim=256, n_heads=4, n_kv_heads=2, ffn_dim=384, n_layers=2)
    args = ModelArgs(dim=256, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=512, ffn_dim=384)
    state = toy_state(cfg, vocab=512, seed=21)
    T.save_checkpoint(str(tmp_path), *T.convert_checkpoint(state, cfg, workers=2))
    dic = T.load_checkpoint(str(tmp_path))
    int8_model = T.convert_bitnet_checkpoint_to_int8(state, cfg)
    model = Transformer.from_checkpoint(args, dic, act="int8")
    tokens = torch.randint(0, args.vocab_size, (2, 24), generator=torch.Generator().manual_seed(22))
    print("[case] toy model from a converted checkpoint", flush=True)
    with torch.inference_mode():
        got = model.forward(tokens.cuda(), model.make_cache(2, 32), torch.arange(24, device="cuda")).float().cpu()
        twin = copy.copy(model)
        twin.tok_embeddings = state["tok_embeddings.weight"].to(torch.bfloat16)
        twin.norm = state["norm.weight"].to(torch.bfloat16)
        twin.layers = []
        names = {"wqkv": "attention.wqkv", "wo": "attention.wo", "w13": "feed_forward.w13", "w2": "feed_forward.w2"}
        norms = {"attention_norm": "attention_norm", "ffn_norm": "ffn_norm", "attn_sub_norm": "attention.attn_sub_norm",
                 "ffn_sub_norm": "feed_forward.ffn_sub_norm"}
        for n, blk in enumerate(model.layers):
            b = copy.copy(blk)
            b.fused = False
            for attr, key in names.items():
                setattr(b, attr, DenseLinearCPU(getattr(blk, attr), "int8", int8_model[f"layers.{n}.{key}.weight"].numpy()))
            for attr, key in norms.items():
                setattr(b, attr, state[f"layers.{n}.{key}.weight"].to(torch.bfloat16))
            twin.layers.append(b)
        want = twin.forward(tokens, twin.make_cache(2, 32), torch.arange(24)).float()
    err, ref = (got - want).abs().max().item(), want.abs().max().item()
    assert err <= 3e-2 * ref, (err, ref)
    assert torch.nn.functional.cosine_similarity(got.flatten(), want.flatten(), dim=0).item() > 0.999
