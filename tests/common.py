"""Shared helpers for the test-suite: small configs and oracle construction."""
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


def make_oracle(cfg, sd, dtype=torch.float32, device="cpu", lean=False):
    return OracleDecoder(oracle_cfg(cfg), sd, dtype=dtype, device=device, lean=lean)
