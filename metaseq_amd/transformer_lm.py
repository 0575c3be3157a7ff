"""Decoder-only language model wrapper with the surface of the reference's BaseModel /
TransformerLanguageModel that generation code touches (metaseq/models/base_model.py:33-198):
``forward`` delegates to the decoder, plus ``max_positions``, ``max_decoder_positions``,
``get_normalized_probs`` and ``make_generation_fast_``."""
from typing import Dict, Optional

import torch
from torch import nn

from .config import OPTConfig
from .transformer_decoder import TransformerDecoder


class TransformerLanguageModel(nn.Module):
    def __init__(self, decoder: TransformerDecoder):
        super().__init__()
        self.decoder = decoder

    @classmethod
    def build_model(cls, cfg: OPTConfig, state_dict: Optional[Dict[str, torch.Tensor]] = None,
                    device="cuda"):
        return cls(TransformerDecoder(cfg, state_dict, device=device))

    def forward(self, src_tokens, **kwargs):
        """metaseq/models/base_model.py:152-168."""
        return self.decoder(src_tokens, **kwargs)

    def forward_decoder(self, prev_output_tokens, **kwargs):
        return self.decoder(prev_output_tokens, **kwargs)

    def extract_features(self, src_tokens, **kwargs):
        return self.decoder.extract_features(src_tokens, **kwargs)

    def output_layer(self, features, **kwargs):
        return self.decoder.output_layer(features, **kwargs)

    def max_positions(self):
        return self.decoder.max_positions()

    def max_decoder_positions(self):
        return self.decoder.max_positions()

    def get_normalized_probs(self, net_output, log_probs: bool):
        """metaseq/models/base_model.py:59-75."""
        return self.decoder.get_normalized_probs(net_output, log_probs)

    def make_generation_fast_(self, **kwargs):
        """metaseq/models/base_model.py:93-135 (puts every sub-module in inference mode)."""
        self.decoder.make_generation_fast_(**kwargs)
        self.eval()

    def load_state_dict(self, state_dict, strict=True, **kw):
        return self.decoder.load_state_dict(state_dict, strict=strict, **kw)

    def state_dict(self, *args, **kwargs):
        sd = {"decoder." + k: v for k, v in self.decoder.state_dict().items()}
        return sd

    @property
    def supported_targets(self):
        return {"future"}
