"""Flat model configuration with the attribute names the reference's decoder reads from
its args namespace (metaseq/models/transformer_decoder.py:73-117,
metaseq/modules/transformer_decoder_layer.py:44-98), and the OPT size table
(metaseq/launcher/opt_job_constants.py:32-45)."""
from dataclasses import dataclass, replace


# head sizes the attention kernels are instantiated for (lanes per key row = head_dim / 8)
SUPPORTED_HEAD_DIMS = (64, 128)


@dataclass
class OPTConfig:
    decoder_layers: int
    decoder_embed_dim: int
    decoder_attention_heads: int
    decoder_ffn_embed_dim: int = 0
    vocab_size: int = 50272  # 50265 tokenizer entries padded to a multiple of 8
    max_target_positions: int = 2048
    padding_idx: int = 1
    eos_idx: int = 2
    activation_fn: str = "relu"
    share_decoder_input_output_embed: bool = True
    decoder_learned_pos: bool = True
    no_scale_embedding: bool = True
    quantize_int8: bool = False  # int8 weight-only for qkv / out_proj / fc1 / fc2

    def __post_init__(self):
        if not self.decoder_ffn_embed_dim:
            self.decoder_ffn_embed_dim = 4 * self.decoder_embed_dim
        if self.decoder_embed_dim % self.decoder_attention_heads:
            raise ValueError("decoder_embed_dim must be divisible by decoder_attention_heads")
        if self.activation_fn != "relu":
            raise NotImplementedError("only --activation-fn relu (OPT) is implemented")
        if not (self.share_decoder_input_output_embed and self.decoder_learned_pos
                and self.no_scale_embedding):
            raise NotImplementedError(
                "only the OPT setup (tied embeddings, learned positions, no embedding scale) "
                "is implemented")

    @property
    def head_dim(self):
        return self.decoder_embed_dim // self.decoder_attention_heads

    def require_supported_head_dim(self):
        """Raised when a decoder is built, before any weight is allocated or packed."""
        if self.head_dim not in SUPPORTED_HEAD_DIMS:
            raise NotImplementedError(
                "head_dim %d (decoder_embed_dim %d / %d heads) is not supported: the attention "
                "kernels are built for head_dim %s" % (
                    self.head_dim, self.decoder_embed_dim, self.decoder_attention_heads,
                    " or ".join(str(h) for h in SUPPORTED_HEAD_DIMS)))


# name -> (layers, embed dim, heads).  OPT-2.7B (32 layers, 2560 / 32 heads = head_dim 80) is
# left out: no attention kernel is built for that head size.
_OPT_SIZES = {
    "125m": (12, 768, 12),
    "350m": (24, 1024, 16),
    "1.3b": (24, 2048, 32),
    "6.7b": (32, 4096, 32),
    "13b": (40, 5120, 40),
    "30b": (48, 7168, 56),
    "66b": (64, 9216, 72),
    "175b": (96, 12288, 96),
}


def opt_config(name: str, **overrides) -> OPTConfig:
    layers, dim, heads = _OPT_SIZES[name.lower()]
    return replace(OPTConfig(layers, dim, heads), **overrides)


def config_from_state_dict(state, heads: int = 0, **overrides) -> OPTConfig:
    """The configuration a reference-named state dict (fp16, or quantised offline) implies:
    layers, widths, vocabulary and position count are read off the tensor shapes.  The number
    of heads is in no shape; it is taken from the OPT size table by (layers, width) unless
    given.  For checkpoints whose own "cfg" entry cannot be read by a loader that executes
    nothing (metaseq/checkpoint_utils.py:540-557 pickles an arbitrary namespace there)."""
    def shape(name):
        for k in (name, "decoder." + name):
            if k in state:
                return tuple(state[k].shape)
        raise KeyError("state dict has no %r" % name)

    layers = 1 + max(int(k.split("layers.")[1].split(".")[0]) for k in state if "layers." in k)
    vocab, dim = shape("embed_tokens.weight")
    positions = shape("embed_positions.weight")[0]
    try:
        ffn = shape("layers.0.fc1.weight")[0]
    except KeyError:
        ffn = shape("layers.0.fc1.qweight")[0]
    if not heads:
        known = {(l, d): h for l, d, h in _OPT_SIZES.values()}
        if (layers, dim) not in known:
            raise ValueError("%d layers of width %d are no OPT size: pass heads=" % (layers, dim))
        heads = known[(layers, dim)]
    padding_idx = overrides.pop("padding_idx", 1)
    # the learned positional table holds padding_idx + 1 unused leading rows
    # (metaseq/modules/learned_positional_embedding.py:23-28)
    cfg = OPTConfig(layers, dim, heads, decoder_ffn_embed_dim=ffn, vocab_size=vocab,
                    max_target_positions=positions - padding_idx - 1, padding_idx=padding_idx)
    return replace(cfg, **overrides)
