"""MI355X-native OPT incremental-decoding forward path (drop-in for metaseq's
TransformerDecoder.forward / SequenceGenerator on one gfx950 GPU)."""
from .config import OPTConfig, config_from_state_dict, opt_config
from .dictionary import Dictionary
from .hub_utils import GeneratorInterface
from .kv_cache import KVCache
from .sequence_generator import SequenceGenerator
from .synthetic import iter_random_state_dict, random_prompts, random_state_dict
from .transformer_decoder import ModelParallelTransformerDecoder, TransformerDecoder
from .transformer_lm import TransformerLanguageModel

__all__ = [
    "OPTConfig", "opt_config", "config_from_state_dict", "Dictionary", "GeneratorInterface", "KVCache", "SequenceGenerator", "random_prompts",
    "random_state_dict", "iter_random_state_dict", "TransformerDecoder", "ModelParallelTransformerDecoder",
    "TransformerLanguageModel",
]
