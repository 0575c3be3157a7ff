"""Request-level front end of the generation path, with the call signature, batching rules and
result records of the reference's ``GeneratorInterface.generate``
(metaseq/hub_utils.py:85-466).

What it does per call: prepend the end-of-sentence token to every prompt and right-pad the
batch (metaseq/tasks/language_modeling.py:287-330), derive the generator's total length limits
from the per-request ``min_tokens`` / ``max_tokens`` (hub_utils.py:300-309), run
``SequenceGenerator`` on the device, then cut every returned row at its first special token,
drop pads, strip the prompt unless ``echo`` and build the ``text`` / ``tokens`` /
``text_offset`` / ``token_scores`` / ``top_logprobs`` record (hub_utils.py:338-413).

The reference builds model, task and BPE from a hydra config and a checkpoint; here the model,
its dictionary and (optionally) a tokenizer are passed in.  The tokenizer needs the two calls
the reference makes on its Hugging Face ``tokenizers`` object: ``decode(ids) -> str`` and
``encode(text).offsets``.  Without one, token ids are rendered as decimal strings.
"""
import time
from typing import List, Optional

import torch

from .sequence_generator import SequenceGenerator


class _IdTokenizer:
    """Stand-in tokenizer: a token is its decimal id, a text is ids joined by single spaces."""

    class _Encoding:
        def __init__(self, ids, offsets):
            self.ids, self.offsets = ids, offsets

    def decode(self, ids):
        return " ".join(str(int(t)) for t in ids)

    def encode(self, text):
        ids, offsets, pos = [], [], 0
        for piece in text.split(" ") if text else []:
            ids.append(int(piece))
            offsets.append((pos, pos + len(piece)))
            pos += len(piece) + 1
        return self._Encoding(ids, offsets)


class GeneratorInterface:
    def __init__(self, model, tgt_dict, tokenizer=None, device="cuda", max_positions=None):
        self.models = [model]
        self.tgt_dict = tgt_dict
        self.bpe = tokenizer if tokenizer is not None else _IdTokenizer()
        self.device = torch.device(device)
        self._max_positions = max_positions
        # hub_utils.py:184-191
        self._pad_token_ind = tgt_dict.pad_index
        self._special_token_inds = {tgt_dict.eos_index, tgt_dict.pad_index, tgt_dict.bos_index,
                                    tgt_dict.unk_index}

    def encode_fn(self, x: str):
        return self.bpe.encode(x.replace("\r\n", "\n").replace("\r", "\n")).ids

    def decode_fn(self, x: List[int]) -> str:
        return self.bpe.decode(x)

    def max_sequence_length(self):
        if self._max_positions is not None:
            return int(self._max_positions)
        return int(min(m.max_positions() for m in self.models))

    def build_batch(self, inputs: List[List[int]]):
        """Prompts with the end-of-sentence token in front, right-padded to a rectangle
        (language_modeling.py:287-330); ``src_lengths`` counts the prepended token."""
        eos, pad = self.tgt_dict.eos_index, self.tgt_dict.pad_index
        width = max(len(t) for t in inputs) + 1
        src = torch.full((len(inputs), width), pad, dtype=torch.long)
        for i, t in enumerate(inputs):
            src[i, 0] = eos
            if len(t):
                src[i, 1:1 + len(t)] = torch.as_tensor(t, dtype=torch.long)
        lengths = torch.tensor([len(t) + 1 for t in inputs], dtype=torch.long)
        return {"net_input": {"src_tokens": src, "src_lengths": lengths}}

    def generate(self, inputs: List[List[int]], min_tokens: List[int] = None,
                 max_tokens: List[int] = None, temperature: float = 1.0, top_p: float = -1.0,
                 logprobs: int = 0, n: int = 1, best_of: Optional[int] = None,
                 echo: bool = False, stop: Optional[List[int]] = None,
                 seed: Optional[int] = None, use_cuda: bool = True, omega_bound: float = 0.3,
                 lambda_decay: float = -1, alpha_presence: float = 0.0,
                 alpha_frequency: float = 0.0, alpha_presence_src: float = 0.0,
                 alpha_frequency_src: float = 0.0, alpha_src_penalty_end_idx: int = -1):
        """Same parameters and return value as the reference (hub_utils.py:195-424): a list
        (one entry per prompt) of lists (``n`` replicas, best cumulative score first) of
        records."""
        if seed:
            torch.manual_seed(seed)
            if torch.cuda.is_available():
                torch.cuda.manual_seed(seed)
        if not use_cuda:
            raise RuntimeError("metaseq_amd: generation runs on the GPU only")
        start_time = time.time()
        if not best_of:
            best_of = n
        assert best_of >= n
        # hub_utils.py:262-274
        sampling_topp = top_p if top_p > 0 else -1
        if temperature == 0:
            temperature, sampling_topp = 1.0, -1
        elif temperature < 0:
            raise ValueError("temperature must be >= 0 and <= 1")

        max_seq_len = self.max_sequence_length()
        batch = self.build_batch(inputs)
        src_tokens = batch["net_input"]["src_tokens"]
        src_lengths = batch["net_input"]["src_lengths"]
        batchsize = src_tokens.size(0)
        lengths = [len(t) for t in inputs]
        if max_tokens is None:
            max_tokens = [max_seq_len] * batchsize
        if min_tokens is None:
            min_tokens = [0] * batchsize
        # hub_utils.py:300-309
        total_max_tokens = min(max_seq_len, max(max_tokens) + int(src_lengths.max()))
        total_min_tokens = max(min_tokens) + int(src_lengths.max())
        generator = SequenceGenerator(
            self.models, self.tgt_dict, beam_size=best_of, max_len_a=0,
            max_len_b=total_max_tokens, min_len=total_min_tokens, temperature=temperature,
            need_logprobs=logprobs > 0, stop=stop, topp=sampling_topp, omega_bound=omega_bound,
            lambda_decay=lambda_decay, alpha_presence=alpha_presence,
            alpha_frequency=alpha_frequency, alpha_presence_src=alpha_presence_src,
            alpha_frequency_src=alpha_frequency_src,
            alpha_src_penalty_end_idx=alpha_src_penalty_end_idx)
        sample = {"net_input": {"src_tokens": src_tokens.to(self.device),
                                "src_lengths": src_lengths.to(self.device)}}
        t0 = time.time()
        translations = generator.generate(self.models, sample)
        self.last_generation_time = time.time() - t0

        all_tokens = translations["tokens"].cpu()[:len(inputs)]
        all_scores = translations["scores"].cpu()[:len(inputs)]
        all_distributions = (translations["distributions"].cpu()[:len(inputs)]
                             if logprobs > 0 else None)
        retval = []
        for i in range(all_tokens.size(0)):
            beams = []
            for j in range(n):
                beams.append(self._record(
                    all_tokens[i, j].tolist(), all_scores[i, j].tolist(),
                    all_distributions[i, j] if logprobs > 0 else None, lengths[i],
                    max_tokens[i], echo, logprobs))
            retval.append(beams)
        self.last_total_time = time.time() - start_time
        return retval

    def _record(self, tokens, scores, distributions, prompt_len, max_tokens, echo, logprobs):
        """One result record (hub_utils.py:344-413)."""
        tokens, scores, distributions = self._filter_special(
            self._pad_token_ind, self._special_token_inds, tokens, scores, distributions)
        if not echo:  # cut off the prompt and its leading end-of-sentence token
            tokens = tokens[prompt_len + 1:][:max_tokens]
            scores = scores[prompt_len + 1:][:max_tokens]
            if logprobs > 0:
                distributions = distributions[prompt_len + 1:][:max_tokens]
        tokens_no_eos = tokens[1:] if echo else tokens
        scores_with_eos = [None] + scores[1:] if echo else scores
        text = self.bpe.decode(tokens_no_eos)
        token_offsets = [s for s, e in self.bpe.encode(text).offsets]
        result = {
            "text": text,
            "tokens": [self.bpe.decode([t]) for t in tokens],
            "text_offset": token_offsets,
            "token_scores": scores_with_eos,
        }
        if logprobs > 0:
            out_logprobs = []
            if distributions.shape[0] > 0:
                top_scores, top_toks = distributions.topk(k=logprobs, dim=-1)
                for sc, tk in zip(top_scores, top_toks):
                    out_logprobs.append({self.bpe.decode([t.item()]): s.item()
                                         for t, s in zip(tk, sc)})
            # no distribution precedes the leading end-of-sentence token
            result["top_logprobs"] = [None] + out_logprobs[1:] if echo else out_logprobs
        else:
            result["top_logprobs"] = None
        return result

    @staticmethod
    def _filter_special(pad_token_ind, special_token_inds, tokens: List[int],
                        scores: List[float], distributions):
        """Drops pads and cuts the sequence at the first special token after position 0
        (hub_utils.py:425-466).  ``distributions`` ([seqlen, vocab] or None) keeps the rows of
        the surviving positions."""
        kept, mask = [], []
        for i, (t, s) in enumerate(zip(tokens, scores)):
            if t == pad_token_ind:
                mask.append(False)
                continue
            if t in special_token_inds and i > 0:
                mask.append(False)
                break
            mask.append(True)
            kept.append((t, s))
        new_tokens, new_scores = zip(*kept)
        if distributions is not None:
            assert len(mask) <= distributions.shape[0], \
                "Mask cannot be larger than the number of tokens in disribution (distributions.shape[0])"
            mask.extend([False] * (distributions.shape[0] - len(mask)))
            distributions = distributions[mask]
        return list(new_tokens), list(new_scores), distributions
