"""Checkpoint-level converter (host logic, no GPU): a random state dict through
ternainfer_amd.convert_checkpoint against the oracle's per-matrix functions, key for key."""
import numpy as np
import pytest
import torch

import ternainfer_amd as T
from oracle import terna_oracle as O

CFG = T.CheckpointShape(dim=128, n_heads=4, n_kv_heads=2, ffn_dim=192, n_layers=2)


def toy_state(cfg=CFG, vocab=256, seed=5, dtype=torch.float32):
    """fp32 by default: the converter computes in the tensors' dtype, and the oracle's ternarisation is fp32."""
    g = torch.Generator().manual_seed(seed)
    r = lambda *shape: (torch.randn(*shape, generator=g) * 0.02).to(dtype)
    state = {}
    for n in range(cfg.n_layers):
        p = f"layers.{n}."
        state[p + "attention.wqkv.weight"] = r(cfg.dim + 2 * cfg.kv_dim, cfg.dim)
        state[p + "attention.wo.weight"] = r(cfg.dim, cfg.dim)
        state[p + "feed_forward.w13.weight"] = r(2 * cfg.ffn_dim, cfg.dim)
        state[p + "feed_forward.w2.weight"] = r(cfg.dim, cfg.ffn_dim)
        for name, width in (("attention_norm", cfg.dim), ("ffn_norm", cfg.dim), ("attention.attn_sub_norm", cfg.dim),
                            ("feed_forward.ffn_sub_norm", cfg.ffn_dim)):
            state[p + name + ".weight"] = (1 + 0.1 * torch.randn(width, generator=g)).to(torch.bfloat16)
    state["tok_embeddings.weight"] = r(vocab, cfg.dim)
    state["output.weight"] = state["tok_embeddings.weight"]
    state["norm.weight"] = torch.ones(cfg.dim, dtype=torch.bfloat16)
    return state


def test_three_dictionaries_key_for_key():
    state = toy_state()
    bf16_model, ternary, non_ternary = T.convert_checkpoint(state, CFG, workers=2)
    linears = [k for k in state if k.endswith(".weight") and state[k].dim() == 2 and "layer" in k]
    assert len(linears) == 4 * CFG.n_layers
    # ternary file: four tensors per linear, the reference's suffixes and dtypes, nothing else
    assert set(ternary) == {k + sfx for k in linears
                            for sfx in ("_compressed_val", "_TileOffsets_global", "_TileOffsets_median", "_bitmap")}
    # non-ternary file: everything that is not a layer matrix except output.weight, plus the weight scales
    want_other = {k for k in state if k not in linears and k != "output.weight"} | \
                 {k.replace("weight", "weight_scale") for k in linears}
    assert set(non_ternary) == want_other
    assert set(bf16_model) == set(state)
    for key in linears:
        w = state[key]
        if "wqkv" in key:
            parts = [w[:CFG.dim], w[CFG.dim:CFG.dim + CFG.kv_dim], w[CFG.dim + CFG.kv_dim:]]
        elif "w13" in key:
            parts = [w[:CFG.ffn_dim], w[CFG.ffn_dim:]]
        else:
            parts = [w]
        tern, scales = zip(*[O.quant_weight_int8(p.float().numpy()) for p in parts])
        want = O.encode(np.concatenate(tern, axis=0))
        got = [ternary[key + sfx].numpy() for sfx in ("_compressed_val", "_TileOffsets_global", "_TileOffsets_median", "_bitmap")]
        for a, b in zip(got, want):
            assert a.dtype == b.dtype and a.shape == b.shape and (a == b).all(), key
        ws = non_ternary[key.replace("weight", "weight_scale")]
        assert ws.dtype == torch.bfloat16 and ws.shape == (4,) and int((ws != 0).sum()) == len(parts)
        for j, sc in enumerate(scales):                       # bf16 arithmetic in the converter: one bf16 step of slack
            assert abs(float(ws[j]) - float(sc)) <= 2.0 ** -7 * float(sc)
        # the dense file holds ternary * scale for every sub-matrix
        dense = bf16_model[key].float().numpy()
        row = 0
        for t, p in zip(tern, parts):
            blk = dense[row:row + t.shape[0]]
            nz = blk[t != 0]
            assert ((blk == 0) == (t == 0)).all() and np.allclose(np.abs(nz), np.abs(nz).flat[0])
            assert (np.sign(blk) == t).all()
            row += t.shape[0]
    for k in want_other - {k.replace("weight", "weight_scale") for k in linears}:
        assert torch.equal(non_ternary[k], state[k])


def test_save_and_load_round_trip(tmp_path):
    state = toy_state(seed=6, dtype=torch.bfloat16)
    parts = T.convert_checkpoint(state, CFG, workers=1)
    T.save_checkpoint(str(tmp_path), *parts)
    merged = T.load_checkpoint(str(tmp_path))
    assert set(merged) == set(parts[1]) | set(parts[2])
    for k, v in {**parts[1], **parts[2]}.items():
        assert merged[k].dtype == v.dtype and torch.equal(merged[k], v)
    dense = T.load_checkpoint(str(tmp_path), bf16=True)
    assert all(torch.equal(dense[k], v) for k, v in parts[0].items())


def test_pairs_to_adjacent_is_the_documented_permutation():
    """'(h l d) i -> (h d l) i' with l = 2: row h*2d + l*d + j moves to h*2d + 2j + l."""
    from ternainfer_amd.convert_utils import _pairs_to_adjacent
    heads, d = 3, 4
    rows = heads * 2 * d
    w = torch.arange(rows, dtype=torch.float32)[:, None].repeat(1, 2)
    got = _pairs_to_adjacent(w, heads)[:, 0].long().tolist()
    want = [0] * rows
    for h in range(heads):
        for l in range(2):
            for j in range(d):
                want[h * 2 * d + 2 * j + l] = h * 2 * d + l * d + j
    assert got == want


def test_convert_back_from_safetensors(tmp_path):
    from safetensors.torch import save_file
    cfg = CFG
    g = torch.Generator().manual_seed(9)
    r = lambda *shape: torch.randn(*shape, generator=g).to(torch.bfloat16)
    src = {"model.embed_tokens.weight": r(64, cfg.dim), "model.norm.weight": r(cfg.dim)}
    for n in range(cfg.n_layers):
        a, f = f"model.layers.{n}.self_attn.", f"model.layers.{n}.mlp."
        src.update({a + "q_proj.weight": r(cfg.dim, cfg.dim), a + "k_proj.weight": r(cfg.kv_dim, cfg.dim),
                    a + "v_proj.weight": r(cfg.kv_dim, cfg.dim), a + "o_proj.weight": r(cfg.dim, cfg.dim),
                    a + "attn_sub_norm.weight": r(cfg.dim), f + "ffn_sub_norm.weight": r(cfg.ffn_dim),
                    f + "gate_proj.weight": r(cfg.ffn_dim, cfg.dim), f + "up_proj.weight": r(cfg.ffn_dim, cfg.dim),
                    f + "down_proj.weight": r(cfg.dim, cfg.ffn_dim),
                    f"model.layers.{n}.input_layernorm.weight": r(cfg.dim),
                    f"model.layers.{n}.post_attention_layernorm.weight": r(cfg.dim)})
    path = str(tmp_path / "m.safetensors")
    save_file(src, path)
    out = T.convert_back(path, cfg)
    assert set(out) == set(toy_state(cfg))
    hd = cfg.dim // cfg.n_heads
    wqkv = out["layers.1.attention.wqkv.weight"]
    q_src = src["model.layers.1.self_attn.q_proj.weight"]
    # head 2, pair 3: source rows (first half, second half) land next to each other
    assert torch.equal(wqkv[2 * hd + 6], q_src[2 * hd + 3]) and torch.equal(wqkv[2 * hd + 7], q_src[2 * hd + hd // 2 + 3])
    assert torch.equal(wqkv[cfg.dim + cfg.kv_dim:], src["model.layers.1.self_attn.v_proj.weight"])
    assert torch.equal(out["layers.0.feed_forward.w13.weight"][cfg.ffn_dim:], src["model.layers.0.mlp.up_proj.weight"])
    assert out["output.weight"] is out["tok_embeddings.weight"] or torch.equal(out["output.weight"], out["tok_embeddings.weight"])
