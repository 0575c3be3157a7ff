"""Tensor-parallel restatement of the reference's decoder forward (fp32, full sequence).

TEST INFRASTRUCTURE ONLY.  It evaluates a list of per-rank state dicts the way the reference's
Megatron layers do on `mp` ranks, with the collectives written out as sums and concatenations
over the list, so that a glued single-part model can be checked against the parts it was
glued from (the invariant the gluing rules must satisfy: same logits).

Followed reference semantics (paths relative to the metaseq tree):
* VocabParallelEmbedding (modules/megatron/mpu/layers.py:220-250): every rank owns a
  contiguous vocabulary range, looks up the ids inside its range, zeroes the others, and the
  partial embeddings are summed (all-reduce).
* ColumnParallelLinear (mpu/layers.py:513-536): rank r holds rows of W and the matching
  bias slice; its output is its slice of the features (qkv_proj, fc1).  For qkv_proj each
  rank's output is split into local thirds K_r | V_r | Q_r (modules/multihead_attention.py:316-319)
  and covers the rank's own heads.
* RowParallelLinear (mpu/layers.py:649-676): rank r holds columns of W, multiplies its
  feature slice, the partial outputs are summed (all-reduce) and the replicated bias is
  added once (out_proj, fc2).
* LayerNorms and the positional table are replicated.
* The tied output projection multiplies by each rank's vocabulary rows and the logits are
  concatenated along the vocabulary (models/transformer_decoder.py:398-428).

Pinned by tests/test_checkpoint_cpu.py: at mp = 1 it must reproduce OracleDecoder exactly,
which is itself pinned against Hugging Face OPT.  For mp > 1 the split of the computation over
ranks is a restatement of the cited reference code with no reference fixture behind it (the
reference ships no multi-part checkpoint or test vector): parity unpinned beyond the facts that
the per-rank pieces sum / concatenate to the mp = 1 result when the parts are cut from one
model, and that every rule is the one metaseq/distributed/stitch_fsdp_ckpt.py:203-339 applies.
"""
from typing import Dict, List

import torch
import torch.nn.functional as F

from .opt_oracle import layer_norm, make_positions


def tp_forward(parts: List[Dict[str, torch.Tensor]], tokens: torch.Tensor, heads: int,
               padding_idx: int = 1) -> torch.Tensor:
    """Logits [B, T, V] of a causal full-sequence forward on `len(parts)` ranks."""
    mp = len(parts)
    w = [{k: v.float() for k, v in p.items() if v.is_floating_point()} for p in parts]
    B, T = tokens.shape
    # vocab-parallel embedding: masked local lookups, summed
    emb = 0
    start = 0
    for r in range(mp):
        E = w[r]["decoder.embed_tokens.weight"]
        n = E.shape[0]
        local = tokens - start
        inside = (local >= 0) & (local < n)
        e = F.embedding(local.clamp(0, n - 1), E) * inside.unsqueeze(-1)
        emb = emb + e
        start += n
    pos = make_positions(tokens, padding_idx)
    x = emb + F.embedding(pos, w[0]["decoder.embed_positions.weight"])
    D = x.shape[-1]
    hd = D // heads
    assert heads % mp == 0
    Hr = heads // mp
    causal = torch.triu(torch.full((T, T), float("-inf")), 1)
    pad = tokens.eq(padding_idx)
    n_layers = 0
    while f"decoder.layers.{n_layers}.fc1.weight" in w[0]:
        n_layers += 1
    for i in range(n_layers):
        p = f"decoder.layers.{i}."
        h = layer_norm(x, w[0][p + "self_attn_layer_norm.weight"],
                       w[0][p + "self_attn_layer_norm.bias"])
        attn = 0
        for r in range(mp):
            kvq = h @ w[r][p + "self_attn.qkv_proj.weight"].t() + w[r][p + "self_attn.qkv_proj.bias"]
            k, v, q = kvq.split(kvq.shape[-1] // 3, dim=-1)      # local thirds
            q = q * hd ** -0.5
            def heads_first(t):
                return t.view(B, T, Hr, hd).transpose(1, 2)       # [B, Hr, T, hd]
            s = heads_first(q) @ heads_first(k).transpose(-1, -2) + causal
            s = s.masked_fill(pad.view(B, 1, 1, T), float("-inf"))
            o = torch.softmax(s, -1) @ heads_first(v)
            o = o.transpose(1, 2).reshape(B, T, Hr * hd)
            attn = attn + o @ w[r][p + "self_attn.out_proj.weight"].t()   # row parallel: partial sums
        x = x + attn + w[0][p + "self_attn.out_proj.bias"]
        h = layer_norm(x, w[0][p + "final_layer_norm.weight"], w[0][p + "final_layer_norm.bias"])
        z = 0
        for r in range(mp):
            u = F.relu(h @ w[r][p + "fc1.weight"].t() + w[r][p + "fc1.bias"])
            z = z + u @ w[r][p + "fc2.weight"].t()
        x = x + z + w[0][p + "fc2.bias"]
    x = layer_norm(x, w[0]["decoder.layer_norm.weight"], w[0]["decoder.layer_norm.bias"])
    return torch.cat([x @ w[r]["decoder.embed_tokens.weight"].t() for r in range(mp)], dim=-1)
