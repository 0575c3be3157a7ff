"""Pins the CPU oracle against material that does not come from the oracle itself:
the reference's own known-answer table, closed forms in float64, brute-force loops,
torch library routines, and Hugging Face's OPT implementation."""
import json
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from metaseq_amd import random_state_dict
from oracle import opt_oracle as O
from tests.common import make_oracle, tiny_cfg

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def test_make_positions_reference_table():
    g = json.load(open(os.path.join(GOLDEN, "make_positions.json")))
    for case in g["cases"]:
        got = O.make_positions(torch.tensor(case["input"]), g["pad"])
        assert got.tolist() == case["output"], case["name"]


def test_layer_norm_closed_form_float64():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(5, 96)).astype(np.float32)
    g = rng.normal(size=96).astype(np.float32)
    b = rng.normal(size=96).astype(np.float32)
    x64 = x.astype(np.float64)
    mu = x64.mean(-1, keepdims=True)
    var = ((x64 - mu) ** 2).mean(-1, keepdims=True)  # biased
    want = (x64 - mu) / np.sqrt(var + 1e-5) * g + b
    got = O.layer_norm(torch.from_numpy(x), torch.from_numpy(g), torch.from_numpy(b)).numpy()
    assert np.abs(got - want).max() < 2e-6
    # a constant row has zero variance: output is exactly beta
    c = torch.full((1, 96), 3.25)
    got = O.layer_norm(c, torch.from_numpy(g), torch.from_numpy(b))
    assert torch.allclose(got[0], torch.from_numpy(b), atol=1e-6)
    # library routine
    lib = F.layer_norm(torch.from_numpy(x), (96,), torch.from_numpy(g), torch.from_numpy(b), 1e-5)
    assert torch.allclose(torch.from_numpy(got.numpy() * 0 + O.layer_norm(
        torch.from_numpy(x), torch.from_numpy(g), torch.from_numpy(b)).numpy()), lib, atol=2e-6)


def _brute_attention(q, k, v, causal_offset):
    """q [T, hd] (already scaled), k/v [S, hd]; query t sees keys 0..causal_offset+t."""
    T, hd = q.shape
    out = np.zeros((T, hd))
    for t in range(T):
        n = causal_offset + t + 1
        s = np.array([sum(q[t, d] * k[j, d] for d in range(hd)) for j in range(n)])
        e = np.exp(s - s.max())
        p = e / e.sum()
        for d in range(hd):
            out[t, d] = sum(p[j] * v[j, d] for j in range(n))
    return out


def test_attention_block_brute_force_and_sdpa():
    """The oracle's attention (K|V|Q split, scaling, head layout, causal mask, cache) against
    python loops and torch's scaled_dot_product_attention, via a 1-layer decoder whose
    other weights are made transparent."""
    cfg = tiny_cfg(layers=1, dim=16, heads=2, vocab=32, max_pos=16)
    sd = random_state_dict(cfg, seed=3, dtype=torch.float32)
    dec = make_oracle(cfg, sd)
    T, B, D, H, hd = 5, 2, 16, 2, 8
    torch.manual_seed(0)
    x = torch.randn(T, B, D)
    inc = {}
    mask = torch.triu(torch.full((T, T), float("-inf")), 1)
    out, bias = dec._attention(0, x, inc, mask, None)
    W = sd["decoder.layers.0.self_attn.qkv_proj.weight"]
    bq = sd["decoder.layers.0.self_attn.qkv_proj.bias"]
    Wk, Wv, Wq = W[:D], W[D:2 * D], W[2 * D:]
    bk, bv, bq_ = bq[:D], bq[D:2 * D], bq[2 * D:]
    Wo = sd["decoder.layers.0.self_attn.out_proj.weight"]
    ctx = torch.zeros(T, B, D)
    for b in range(B):
        for h in range(H):
            sl = slice(h * hd, (h + 1) * hd)
            q = ((x[:, b] @ Wq.t() + bq_)[:, sl] * hd ** -0.5).double().numpy()
            k = (x[:, b] @ Wk.t() + bk)[:, sl].double().numpy()
            v = (x[:, b] @ Wv.t() + bv)[:, sl].double().numpy()
            ctx[:, b, sl] = torch.from_numpy(_brute_attention(q, k, v, 0)).float()
            sd_out = F.scaled_dot_product_attention(
                torch.from_numpy(q)[None], torch.from_numpy(k)[None], torch.from_numpy(v)[None],
                is_causal=True, scale=1.0)[0]
            assert torch.allclose(sd_out.float(), ctx[:, b, sl], atol=1e-5)
    want = ctx @ Wo.t()
    assert torch.allclose(out, want, atol=1e-5)
    # incremental step: one more token attends to the 5 cached keys plus itself
    x1 = torch.randn(1, B, D)
    out1, _ = dec._attention(0, x1, inc, None, None)
    xa = torch.cat([x, x1], 0)
    for b in range(B):
        row = torch.zeros(D)
        for h in range(H):
            sl = slice(h * hd, (h + 1) * hd)
            q = ((x1[:, b] @ Wq.t() + bq_)[:, sl] * hd ** -0.5).double().numpy()
            k = (xa[:, b] @ Wk.t() + bk)[:, sl].double().numpy()
            v = (xa[:, b] @ Wv.t() + bv)[:, sl].double().numpy()
            row[sl] = torch.from_numpy(_brute_attention(q, k, v, T)).float()[0]
        assert torch.allclose(out1[0, b], row @ Wo.t(), atol=1e-5)
    key = dec.layer_ids[0] + ".attn_state"
    assert inc[key]["prev_key"].shape == (B, H, T + 1, hd)


@pytest.mark.parametrize("pad_rows", [False, True])
def test_incremental_equals_full_recompute(pad_rows):
    cfg = tiny_cfg(layers=2, dim=64, heads=4, vocab=96, max_pos=32)
    sd = random_state_dict(cfg, seed=11, dtype=torch.float32)
    dec = make_oracle(cfg, sd)
    g = torch.Generator().manual_seed(5)
    toks = torch.randint(4, 96, (3, 12), generator=g)
    toks[:, 0] = 2
    if pad_rows:
        toks[1, 5:8] = 1  # pads in the middle of the prompt region
    inc = {}
    P = 8
    logits = dec(toks[:, :P], incremental_state=inc)[0]
    full = dec(toks[:, :P])[0]
    assert torch.equal(logits, full)
    for t in range(P, 12):
        step = dec(toks[:, :t + 1], incremental_state=inc)[0]
        ref = dec(toks[:, :t + 1])[0][:, -1:]
        assert step.shape == (3, 1, 96)
        assert torch.allclose(step, ref, atol=2e-5), t


def _hf_model(cfg, sd):
    from transformers import OPTConfig as HFConfig
    from transformers import OPTForCausalLM

    D = cfg.decoder_embed_dim
    hc = HFConfig(vocab_size=cfg.vocab_size, hidden_size=D, num_hidden_layers=cfg.decoder_layers,
                  ffn_dim=cfg.decoder_ffn_embed_dim, num_attention_heads=cfg.decoder_attention_heads,
                  max_position_embeddings=cfg.max_target_positions, do_layer_norm_before=True,
                  word_embed_proj_dim=D, activation_function="relu", enable_bias=True,
                  layer_norm_elementwise_affine=True, dropout=0.0, attention_dropout=0.0,
                  layerdrop=0.0, pad_token_id=1, bos_token_id=2, eos_token_id=2,
                  tie_word_embeddings=True)
    hc._attn_implementation = "eager"
    m = OPTForCausalLM(hc).eval().float()
    hsd = {}
    hsd["model.decoder.embed_tokens.weight"] = sd["decoder.embed_tokens.weight"]
    hsd["lm_head.weight"] = sd["decoder.embed_tokens.weight"]
    hsd["model.decoder.embed_positions.weight"] = sd["decoder.embed_positions.weight"]
    hsd["model.decoder.final_layer_norm.weight"] = sd["decoder.layer_norm.weight"]
    hsd["model.decoder.final_layer_norm.bias"] = sd["decoder.layer_norm.bias"]
    for i in range(cfg.decoder_layers):
        s, d = f"decoder.layers.{i}.", f"model.decoder.layers.{i}."
        W, b = sd[s + "self_attn.qkv_proj.weight"], sd[s + "self_attn.qkv_proj.bias"]
        for j, nm in enumerate(["k_proj", "v_proj", "q_proj"]):  # rows K | V | Q
            hsd[d + f"self_attn.{nm}.weight"] = W[j * D:(j + 1) * D]
            hsd[d + f"self_attn.{nm}.bias"] = b[j * D:(j + 1) * D]
        for a, bname in [("self_attn.out_proj", "self_attn.out_proj"),
                         ("self_attn_layer_norm", "self_attn_layer_norm"),
                         ("final_layer_norm", "final_layer_norm"), ("fc1", "fc1"), ("fc2", "fc2")]:
            hsd[d + bname + ".weight"] = sd[s + a + ".weight"]
            hsd[d + bname + ".bias"] = sd[s + a + ".bias"]
    missing, unexpected = m.load_state_dict(hsd, strict=False)
    assert not unexpected, unexpected
    assert all("lm_head" in k or "embed_tokens" in k for k in missing), missing
    return m


def test_whole_decoder_matches_huggingface_opt():
    """The relation the reference's gpu_tests/test_hf_compatibility.py:128-155 asserts
    (metaseq forward == HF OPT forward), here at fp32 with seeded random weights and a far
    tighter tolerance than its atol=1e-1."""
    cfg = tiny_cfg(layers=3, dim=64, heads=4, vocab=200, max_pos=48)
    sd = random_state_dict(cfg, seed=21, dtype=torch.float32, std=0.2)
    dec = make_oracle(cfg, sd)
    hf = _hf_model(cfg, sd)
    g = torch.Generator().manual_seed(9)
    toks = torch.randint(4, 200, (3, 20), generator=g)
    toks[:, 0] = 2
    toks[1, 15:] = 1  # right-padded rows, as the service batches them
    toks[2, 9:] = 1
    with torch.no_grad():
        want = hf(input_ids=toks, attention_mask=toks.ne(1).long()).logits
    got = dec(toks)[0]
    valid = toks.ne(1)
    assert (got[valid] - want[valid]).abs().max() < 2e-4
    assert torch.equal(got[valid].argmax(-1), want[valid].argmax(-1))
    # incremental decoding against HF's own cache
    with torch.no_grad():
        P = 8
        inc = {}
        out = hf(input_ids=toks[:1, :P], use_cache=True)
        o = dec(toks[:1, :P], incremental_state=inc)[0]
        assert (o - out.logits).abs().max() < 2e-4
        past = out.past_key_values
        for t in range(P, 14):
            out = hf(input_ids=toks[:1, t:t + 1], past_key_values=past, use_cache=True)
            past = out.past_key_values
            o = dec(toks[:1, :t + 1], incremental_state=inc)[0]
            assert (o - out.logits).abs().max() < 2e-4, t


def test_fp16_faithful_mode_close_to_fp32_and_rounds():
    cfg = tiny_cfg(layers=2, dim=64, heads=4, vocab=96, max_pos=32)
    sd = random_state_dict(cfg, seed=2, dtype=torch.float16)
    d32 = make_oracle(cfg, sd, torch.float32)
    d16 = make_oracle(cfg, sd, torch.float16)
    toks = torch.randint(4, 96, (2, 10), generator=torch.Generator().manual_seed(1))
    a, b = d32(toks)[0], d16(toks)[0]
    assert torch.equal(b, b.half().float())  # logits are fp16 values
    assert (a - b).abs().max() < 2e-2


def test_quantize_int8_closed_form():
    g = torch.Generator().manual_seed(4)
    w = (torch.randn(6, 40, generator=g) * 0.02).half()
    q, s = O.quantize_int8(w)
    assert q.dtype == torch.int8 and s.dtype == torch.float16
    for j in range(6):
        row = w[j].double()
        sj = float(torch.tensor(float(row.abs().max()) / 127.0).half())
        assert float(s[j]) == sj
        for i in range(40):
            want = max(-127, min(127, int(np.rint(float(row[i]) / sj))))
            # rint ties: the fp32 division may land within 1 ulp of .5 - allow neither side
            assert abs(int(q[j, i]) - float(row[i]) / sj) <= 0.5 + 1e-3
            assert abs(int(q[j, i]) - want) <= 1
    deq = O.dequantize_int8(q, s)
    assert (deq.float() - w.float()).abs().max() <= float(s.float().max()) * 0.51
    # the largest-magnitude entry of each row maps to +-127
    assert torch.equal(q.abs().amax(1), torch.full((6,), 127, dtype=torch.int8))


def test_lean_mode_changes_no_value():
    """lean=True (weights and history stored in fp16, attention walked over batch rows in
    chunks) is a memory layout of the same arithmetic: logits and tokens equal the plain
    oracle's bit for bit, with a padded row, prefill and incremental steps."""
    from metaseq_amd import random_prompts, random_state_dict
    from oracle.opt_oracle import greedy_generate
    from tests.common import make_oracle, tiny_cfg
    cfg = tiny_cfg(layers=3, dim=128, heads=2, vocab=128, max_pos=64)
    sd = random_state_dict(cfg, seed=7, dtype=torch.float16)
    plain = make_oracle(cfg, sd, torch.float16)
    lean = make_oracle(cfg, sd, torch.float16, lean=True)
    lean.attn_chunk_bytes = 2 * 12 * 12 * 4  # one batch row per chunk
    toks = random_prompts(cfg, 3, 20, seed=5)
    toks[1, 15:] = 1
    a = greedy_generate(plain, toks[:, :12], max_len_b=30, min_len=29, return_step_logits=True)
    b = greedy_generate(lean, toks[:, :12], max_len_b=30, min_len=29, return_step_logits=True)
    assert torch.equal(a["tokens"], b["tokens"]) and torch.equal(a["scores"], b["scores"])
    for x, y in zip(a["step_logits"], b["step_logits"]):
        assert torch.equal(x, y)
    assert torch.equal(plain(toks)[0], lean(toks)[0])


def test_given_token_embeddings_replace_the_lookup():
    """Handing the oracle the looked-up embeddings changes nothing (prefill and decode step);
    handing it other rows changes exactly what a changed embedding table would."""
    cfg = tiny_cfg(layers=2, dim=32, heads=2, vocab=40, max_pos=16)
    sd = random_state_dict(cfg, seed=4, dtype=torch.float32)
    dec = make_oracle(cfg, sd)
    toks = torch.tensor([[2, 7, 9, 11], [2, 5, 1, 1]])
    E = sd["decoder.embed_tokens.weight"]
    a_inc, b_inc = {}, {}
    a = dec(toks[:, :3], incremental_state=a_inc)[0]
    b = dec(toks[:, :3], incremental_state=b_inc, token_embeddings=E[toks[:, :3]])[0]
    assert torch.equal(a, b)
    a = dec(toks, incremental_state=a_inc)[0]
    b = dec(toks, incremental_state=b_inc, token_embeddings=E[toks[:, -1:]])[0]
    assert torch.equal(a, b)
    # other rows: the same as a table whose rows for these ids were replaced
    other = torch.randn(2, 3, 32, generator=torch.Generator().manual_seed(1)) * 0.02
    sd2 = dict(sd)
    E2 = E.clone()
    ids = torch.tensor([[30, 31, 32], [33, 34, 35]])          # unused ids stand for the new rows
    E2[ids] = other
    sd2["decoder.embed_tokens.weight"] = E2
    t2 = torch.cat([toks[:, :1] * 0 + ids[:, :1], ids[:, 1:]], 1)
    want = make_oracle(cfg, sd2).extract_features(t2)[0]
    got = dec.extract_features(t2, token_embeddings=other)[0]
    assert torch.allclose(got, want, atol=1e-6)
