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

import numpy as np
import torch

from .sequence_generator import SequenceGenerator


class TopRows:
    """What is kept of a row's per-position distributions when only the best entries are
    reported: ``values`` / ``ids`` [positions, k], most likely first.  Indexable by position
    like the dense [positions, vocab] array it stands for."""

    def __init__(self, values, ids):
        self.values, self.ids = np.asarray(values, dtype=np.float64), np.asarray(ids, np.int64)
        self.shape = self.values.shape

    @classmethod
    def from_pairs(cls, pairs, k):
        """``pairs``: per position (values, ids) lists of k entries, or empty lists for a
        position without a prediction (stored as -inf / id 0)."""
        values = np.full((len(pairs), k), -np.inf)
        ids = np.zeros((len(pairs), k), dtype=np.int64)
        for i, (v, t) in enumerate(pairs):
            if len(v):
                values[i], ids[i] = v, t
        return cls(values, ids)

    def __getitem__(self, sel):
        return TopRows(self.values[sel], self.ids[sel])


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
        # handed to every SequenceGenerator this interface builds (see its noise_fn)
        self.noise_fn = None
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
        generator.noise_fn = self.noise_fn
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
        """One result record with the reference's fields (hub_utils.py:344-413): ``text``,
        per-token strings, character offsets, scores and, on request, the ``logprobs`` most
        likely alternatives per position.

        After the special-token cut the row holds [eos, prompt..., continuation...].  The
        reported window is the whole row with ``echo`` and the continuation (capped at the
        request's own ``max_tokens``) without; with ``echo`` the leading end-of-sentence token
        shows up among the token strings but has no score, no alternatives and no text."""
        tokens, scores, distributions = self._filter_special(
            self._pad_token_ind, self._special_token_inds, tokens, scores, distributions)
        lo = 0 if echo else prompt_len + 1
        hi = len(tokens) if echo else min(len(tokens), lo + max_tokens)
        window = slice(lo, max(lo, hi))
        shown, shown_scores = tokens[window], scores[window]
        lead = 1 if echo else 0  # positions at the front that carry no prediction
        text = self.bpe.decode(shown[lead:])
        record = {
            "text": text,
            "tokens": [self.bpe.decode([t]) for t in shown],
            "text_offset": [begin for begin, _ in self.bpe.encode(text).offsets],
            "token_scores": [None] * lead + shown_scores[lead:],
            "top_logprobs": None,
        }
        if logprobs > 0:
            best = self._alternatives(distributions[window], logprobs)
            record["top_logprobs"] = [None] * lead + best[lead:]
        return record

    def _alternatives(self, rows, k):
        """Per position, the k most likely tokens as {token string: log-probability}."""
        if rows.shape[0] == 0:
            return []
        if isinstance(rows, TopRows):
            values, ids = rows.values[:, :k], rows.ids[:, :k]
        else:
            values, ids = torch.as_tensor(rows).topk(k, dim=-1)
        return [{self.bpe.decode([i]): v for i, v in zip(id_row, value_row)}
                for id_row, value_row in zip(ids.tolist(), values.tolist())]

    @staticmethod
    def _filter_special(pad_token_ind, special_token_inds, tokens: List[int],
                        scores: List[float], distributions):
        """The part of a generated row that is reported (hub_utils.py:425-466): the row ends
        before the first special token that is not a pad and not at position 0, and pads in
        front of that point are dropped.  ``distributions`` ([positions, vocab] array or tensor,
        or None) keeps the rows of the surviving positions."""
        ids = np.asarray(tokens, dtype=np.int64)
        enders = np.isin(ids, [t for t in special_token_inds if t != pad_token_ind])
        enders[:1] = False
        end = int(enders.argmax()) if enders.any() else ids.size
        keep = np.flatnonzero(ids[:end] != pad_token_ind).tolist()
        if distributions is not None:
            examined = min(end + 1, ids.size)
            if examined > distributions.shape[0]:
                raise AssertionError("%d positions were generated but only %d distributions "
                                     "were recorded" % (examined, distributions.shape[0]))
            distributions = distributions[keep]
        return [tokens[i] for i in keep], [scores[i] for i in keep], distributions
