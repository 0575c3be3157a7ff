"""Seeded random-init OPT weights and prompts (there are no checkpoints offline).

Parameter names and shapes are the reference's state-dict layout at tensor-parallel size 1
(metaseq/scripts/convert_metaseq_ft.py:74-90; qkv_proj rows are K | V | Q,
metaseq/modules/multihead_attention.py:188-197, 316-319).  Every tensor is drawn in a fixed
order from one generator: matrices, embeddings and biases ~ N(0, 0.02), LayerNorm weight
1 + N(0, 0.02), and the padding rows of both embedding tables are zero as in the reference
(metaseq/modules/positional_embedding.py:46-47).
"""
from typing import Dict, Iterator, Tuple

import torch

from .config import OPTConfig


def iter_random_state_dict(cfg: OPTConfig, seed: int = 1234, dtype=torch.float16,
                           device="cpu", std: float = 0.02) -> Iterator[Tuple[str, torch.Tensor]]:
    """Yields (name, tensor) one at a time, in the fixed drawing order, so that a model far
    larger than the spare memory can be filled without ever holding a second copy of it."""
    device = torch.device(device)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)

    def normal(*shape, mean=0.0):
        t = torch.empty(*shape, dtype=torch.float32, device=device)
        t.normal_(mean, std, generator=gen)
        return t.to(dtype)

    D, F, V = cfg.decoder_embed_dim, cfg.decoder_ffn_embed_dim, cfg.vocab_size
    yield "decoder.version", torch.tensor([3.0])
    e = normal(V, D)
    e[cfg.padding_idx].zero_()
    yield "decoder.embed_tokens.weight", e
    del e
    p = normal(cfg.max_target_positions + cfg.padding_idx + 1, D)
    p[cfg.padding_idx].zero_()
    yield "decoder.embed_positions.weight", p
    del p
    for i in range(cfg.decoder_layers):
        pre = f"decoder.layers.{i}."
        yield pre + "self_attn_layer_norm.weight", normal(D, mean=1.0)
        yield pre + "self_attn_layer_norm.bias", normal(D)
        yield pre + "self_attn.qkv_proj.weight", normal(3 * D, D)
        yield pre + "self_attn.qkv_proj.bias", normal(3 * D)
        yield pre + "self_attn.out_proj.weight", normal(D, D)
        yield pre + "self_attn.out_proj.bias", normal(D)
        yield pre + "final_layer_norm.weight", normal(D, mean=1.0)
        yield pre + "final_layer_norm.bias", normal(D)
        yield pre + "fc1.weight", normal(F, D)
        yield pre + "fc1.bias", normal(F)
        yield pre + "fc2.weight", normal(D, F)
        yield pre + "fc2.bias", normal(D)
    yield "decoder.layer_norm.weight", normal(D, mean=1.0)
    yield "decoder.layer_norm.bias", normal(D)


def random_state_dict(cfg: OPTConfig, seed: int = 1234, dtype=torch.float16,
                      device="cpu", std: float = 0.02) -> Dict[str, torch.Tensor]:
    return dict(iter_random_state_dict(cfg, seed, dtype, device, std))


def random_prompts(cfg: OPTConfig, batch: int, prompt_len: int, seed: int = 4321,
                   device="cpu") -> torch.Tensor:
    """[batch, 1 + prompt_len] ids: an EOS followed by uniform ids in [4, vocab) - the
    reference's inference dataset prepends EOS to every prompt
    (metaseq/tasks/language_modeling.py:303-311)."""
    gen = torch.Generator()
    gen.manual_seed(seed)
    ids = torch.randint(4, cfg.vocab_size, (batch, prompt_len), generator=gen, dtype=torch.long)
    eos = torch.full((batch, 1), cfg.eos_idx, dtype=torch.long)
    return torch.cat([eos, ids], dim=1).to(device)
