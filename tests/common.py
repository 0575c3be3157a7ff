"""Shared helpers for the test-suite: small configs and oracle construction."""
import math

import torch

from metaseq_amd import OPTConfig, random_state_dict
from oracle.opt_oracle import OracleConfig, OracleDecoder


def tiny_cfg(layers=2, dim=128, heads=2, vocab=128, max_pos=64, ffn=0):
    return OPTConfig(layers, dim, heads, decoder_ffn_embed_dim=ffn, vocab_size=vocab,
                     max_target_positions=max_pos)


def oracle_cfg(cfg):
    return OracleConfig(cfg.decoder_layers, cfg.decoder_embed_dim, cfg.decoder_attention_heads,
                        cfg.decoder_ffn_embed_dim, cfg.vocab_size, cfg.max_target_positions,
                        cfg.padding_idx, cfg.eos_idx)


def make_oracle(cfg, sd, dtype=torch.float32, device="cpu", lean=False, store_dtype=None):
    return OracleDecoder(oracle_cfg(cfg), sd, dtype=dtype, device=device, lean=lean,
                         store_dtype=store_dtype)


def assert_tokens_match_up_to_ties(got, want, step_logits, n0, ulps=2, pad=1, eos=2,
                                   prefill_index=None):
    """Greedy rows must be identical, except that a row may leave the oracle's path at a
    numerical tie: at the first position where it differs, the oracle's own logit of the token
    the HIP path chose lies within ``ulps`` fp16 ulps of the oracle's best (the fp32 summation
    order then decides).  ``step_logits[i]`` are the oracle's logits of the forward that chose
    position ``n0 + i``; ``prefill_index[r]`` is the position of the prefill logits that
    predicts row r's first token (the last one unless the prompt is right-padded).  Returns the
    rows that diverged."""
    got, want = got.cpu(), want.cpu()
    rows = (got != want).any(dim=1).nonzero().flatten().tolist()
    for r in rows:
        t = int((got[r] != want[r]).nonzero()[0])
        at = prefill_index[r] if (t == n0 and prefill_index is not None) else -1
        lg = step_logits[t - n0][r, at].float().cpu().clone()
        lg[pad] = lg[eos] = float("-inf")
        top = float(lg.max())
        ulp = 2.0 ** (math.floor(math.log2(abs(top))) - 10) if top != 0 else 2.0 ** -24
        short = (top - float(lg[int(got[r, t])])) / ulp
        print("row %d leaves the oracle's path at position %d, %.1f ulp below the oracle's best"
              % (r, t, short), flush=True)
        assert short <= ulps + 1e-3, (r, t, short)
    return rows
