"""Generation loop with the constructor, call signature and return value of the reference's
``SequenceGenerator`` (metaseq/sequence_generator.py:26-534).

Greedy decoding is the fast path: the reference makes ~6 full-vocabulary fp32 passes and two
device-to-host syncs per step; here one kernel per step does log-sum-exp, masking, arg-max,
token/score write-back and the finished-row update on the device, and the host only syncs
once end-of-sequence becomes possible (step >= min_len).

Nucleus (top-p) sampling, factual-nucleus decay, the repetition penalties and ``need_logprobs``
take the general path: one kernel per step (msa_sample_topp_f16) applies the reference's masks
and penalties (:271-293, :478-523), writes the step's masked fp32 log-probabilities straight
into the ``distributions`` buffer when they are wanted (:301-303), finds the nucleus without
sorting and draws from it (or takes the arg-max).  Factual-nucleus state is kept per row (the
reference's indexing only works at beam_size 1, where the two agree), and prompt-token counts of
a replica row come from its own prompt (the reference indexes past the prompt batch when
beam_size > 1).
"""
import ctypes
from typing import Dict, List, Optional

import torch
from torch import nn

from . import _capi
from ._capi import check, ptr


class _FinishWatch:
    """"Have all rows finished?", asked of the device without making it wait: ``post`` queues
    the test of the flags as they stand and its copy to pinned host memory; ``all_finished``
    waits for that copy alone (not for work queued after it) and returns the answer."""

    def __init__(self, finished: torch.Tensor):
        self.finished = finished
        self.host = torch.zeros(1, dtype=torch.bool, pin_memory=True)
        self.event = torch.cuda.Event()
        self.posted = False

    def post(self):
        self.host.copy_(self.finished.all().view(1), non_blocking=True)
        self.event.record()
        self.posted = True

    def all_finished(self) -> bool:
        if not self.posted:
            return False
        self.event.synchronize()
        self.posted = False
        return bool(self.host[0])


class SequenceGenerator(nn.Module):
    def __init__(self, models, tgt_dict, beam_size: int = 1, max_len_a: int = 0,
                 max_len_b: int = 200, min_len: int = 1, temperature: float = 1.0,
                 need_logprobs: bool = False, stop: Optional[List[int]] = None,
                 topp: float = -1, profile=False, omega_bound: float = 0.3,
                 lambda_decay: float = -1, alpha_presence: float = 0.0,
                 alpha_frequency: float = 0.0, alpha_presence_src: float = 0.0,
                 alpha_frequency_src: float = 0.0, alpha_src_penalty_end_idx: int = -1,
                 use_graph: bool = False):
        super().__init__()
        # replay each decode step (selection + forward) as one captured hipGraph where possible
        self.use_graph = use_graph
        self.model = models[0] if isinstance(models, (list, tuple)) else models
        self.tgt_dict = tgt_dict
        self.pad = tgt_dict.pad()
        self.unk = tgt_dict.unk()
        self.eos = tgt_dict.eos()
        self.vocab_size = len(tgt_dict)
        self.beam_size = min(beam_size, self.vocab_size - 1)
        self.max_len_a = max_len_a
        self.max_len_b = max_len_b
        self.min_len = min_len
        self.need_logprobs = need_logprobs
        self.stop = list(stop) if stop is not None else []
        if topp is None:
            topp = 0.0
        self.sampling_topp = max(0, topp)
        self.temperature = temperature
        assert temperature >= 0, "--temperature must be >=0"
        if len(self.stop) > 14:
            raise ValueError("at most 14 stop tokens are supported")
        # factual nucleus (:107-116) and repetition penalties (:118-123)
        self.lambda_decay = lambda_decay
        self.omega_bound = float(omega_bound)
        self.full_stop_list = [tgt_dict.index(w) for w in [".", "?", "!"]]
        if lambda_decay > 0 and all(i == self.unk for i in self.full_stop_list):
            # the decayed nucleus is only ever reset at a full stop: with a dictionary that
            # cannot name ".", "?" and "!" it would silently decay to omega_bound for good
            raise ValueError(
                "factual-nucleus sampling (lambda_decay > 0) needs a dictionary that resolves "
                "'.', '?' and '!' to token ids; this one maps them all to <unk>")
        self.alpha_presence = alpha_presence
        self.alpha_frequency = alpha_frequency
        self.alpha_presence_src = alpha_presence_src
        self.alpha_frequency_src = alpha_frequency_src
        self.alpha_src_penalty_end_idx = alpha_src_penalty_end_idx
        self.sampling = not (self.temperature == 0.0 or self.sampling_topp == 0.0)
        self.penalties = max(alpha_presence, alpha_frequency) > 0
        self.penalties_src = max(alpha_presence_src, alpha_frequency_src) > 0
        self.model.eval()
        self.profile = profile
        # noise_fn(step, rows, vocab) -> fp32 [rows, vocab] device tensor of independent Exp(1)
        # numbers for the draw of that step; None: torch's device generator (torch.manual_seed)
        self.noise_fn = None

    def cuda(self):
        self.model.cuda()
        return self

    @torch.no_grad()
    def forward(self, sample, prefix_tokens=None, bos_token=None):
        return self._generate(sample, prefix_tokens, bos_token=bos_token)

    @torch.no_grad()
    def generate(self, models, sample, **kwargs):
        return self._generate(sample, **kwargs)

    # ------------------------------------------------------------------
    def _banned(self, step, min_len):
        """Ids that cannot be chosen at ``step``: pad always, eos and the stop tokens before the
        minimum length (metaseq/sequence_generator.py:272-279)."""
        banned = [self.pad]
        if step < min_len:
            banned += [self.eos] + self.stop
        return banned

    def _select(self, lib, logits2d, step, min_len, max_len, finished, tokens, scores,
                len_dev=None):
        """Fused log-softmax + masks + arg-max + bookkeeping for one step
        (metaseq/sequence_generator.py:272-308).  With ``len_dev`` the output column is read
        from the device (``step`` then only selects the masks)."""
        banned = self._banned(step, min_len)
        B, V = logits2d.shape
        arr = (ctypes.c_int32 * len(banned))(*banned)
        stop = (ctypes.c_int32 * max(1, len(self.stop)))(*self.stop)
        col = 0 if len_dev is not None else step
        tok = tokens[:, col]
        sc = scores[:, col]
        check(lib.msa_greedy_select_f16(
            ptr(logits2d), logits2d.stride(0), B, V, float(self.temperature), arr, len(banned),
            stop, len(self.stop), ptr(finished), None, int(step >= max_len - 1), self.eos,
            ptr(tok), tokens.stride(0), ptr(sc), scores.stride(0), ptr(len_dev),
            _capi.stream_ptr()))

    @staticmethod
    def static_state(decoder, cache, tokens, scores, finished, step_logits):
        """State of graph-replayed decoding: fixed-address buffers plus the device-side per-row
        lengths (= positions already in ``cache``; all rows equal here, and the next token goes
        to that column of ``tokens``)."""
        return {"graphs": {}, "decoder": decoder, "cache": cache, "tokens": tokens,
                "scores": scores, "finished": finished,
                "logits": step_logits.contiguous().clone(),
                "len_dev": torch.full((tokens.shape[0],), cache.length, dtype=torch.int32,
                                      device=tokens.device)}

    def _graph_body(self, lib, st, step, min_len, max_len):
        """One decode step with nothing step-dependent in its launch arguments: select the token
        for column *len_dev from the static logits, run the forward over the history including
        it, advance the device-side length."""
        self._select(lib, st["logits"], step, min_len, max_len, st["finished"], st["tokens"],
                     st["scores"], st["len_dev"])
        st["decoder"].decode_step_static(st["tokens"], st["cache"], st["len_dev"], st["logits"])
        check(lib.msa_advance_len(ptr(st["len_dev"]), None, st["len_dev"].numel(), 1,
                                  _capi.stream_ptr()))

    def _graph_step(self, lib, st, step, min_len, max_len):
        """Runs the step through a captured graph; the first step of each masking regime
        (before / after min_len) runs eagerly as the warm-up and is then captured."""
        key = step < min_len
        g = st["graphs"].get(key)
        if g is None:
            self._graph_body(lib, st, step, min_len, max_len)  # eager: a real step
            torch.cuda.current_stream().synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                self._graph_body(lib, st, step, min_len, max_len)  # recorded, not executed
            st["graphs"][key] = g
        else:
            g.replay()
        st["cache"].length += 1

    def _generate(self, sample: Dict[str, Dict[str, torch.Tensor]], prefix_tokens=None,
                  bos_token=None):
        lib = _capi.load()
        incremental_states: Dict = {}
        net_input = sample["net_input"]
        if "src_tokens" not in net_input:
            raise Exception("expected src_tokens in net input")
        src_tokens = net_input["src_tokens"]
        if not src_tokens.is_cuda:
            raise RuntimeError("metaseq_amd: src_tokens must live on the GPU")
        src_lengths = (src_tokens.ne(self.eos) & src_tokens.ne(self.pad)).long().sum(dim=1)
        bsz, src_len = src_tokens.size()[:2]
        beam_size = self.beam_size
        dev = src_tokens.device

        max_len = int(min(self.model.max_decoder_positions(), self.max_len_b or 1e99))
        min_len = min(max_len, self.min_len or 0)
        assert min_len <= max_len, "min_len cannot be larger than max_len, please adjust these!"
        start_step = src_tokens.shape[1]
        if start_step > max_len:
            raise ValueError("prompt length %d exceeds max_len %d" % (start_step, max_len))
        BB = bsz * beam_size

        scores = torch.zeros(BB, max_len, device=dev, dtype=torch.float32)
        tokens = torch.full((BB, max_len), self.pad, device=dev, dtype=torch.long)
        tokens[:, :start_step] = src_tokens.repeat_interleave(beam_size, 0)
        rep_lengths = src_lengths.repeat_interleave(beam_size, 0)
        all_lprobs = None
        if self.need_logprobs:
            all_lprobs = torch.zeros(BB, max_len, self.vocab_size, device=dev,
                                     dtype=torch.float32)

        decoder = self.model.decoder
        old_cap = getattr(decoder, "kv_cache_capacity", None)
        decoder.kv_cache_capacity = max_len
        try:
            # ---- prefill over all forced tokens (:223-230) ----
            logits = self.model(tokens[:, :start_step], incremental_state=incremental_states)[0]
            T, V = logits.shape[1], logits.shape[2]
            flat = logits.view(BB * T, V)
            stream = _capi.stream_ptr()
            # log-prob of every prompt token given its prefix (:252-258)
            if start_step > 1:
                target = torch.zeros(BB, T, dtype=torch.long, device=dev)
                target[:, :-1] = tokens[:, 1:start_step]
                lp = torch.empty(BB, T, dtype=torch.float32, device=dev)
                check(lib.msa_target_logprob_f16(ptr(flat), flat.stride(0), BB * T, V,
                                                 float(self.temperature), ptr(target), ptr(lp),
                                                 stream))
                scores[:, 1:start_step] = lp[:, :-1]
            # scores after each row's own prompt are reset (:262-266)
            col = torch.arange(max_len, device=dev).unsqueeze(0)
            scores.masked_fill_(col > rep_lengths.unsqueeze(1), 0.0)
            if all_lprobs is not None and start_step > 1:
                # the distributions of the prompt positions (:247-250), fp32 rows written in place
                dst = all_lprobs[:, 1]
                check(lib.msa_log_softmax_f16(ptr(flat), T * flat.stride(0), flat.stride(0), BB,
                                              start_step - 1, V, float(self.temperature), ptr(dst),
                                              all_lprobs.stride(0), all_lprobs.stride(1), stream))
            # the row that predicts each sample's first free token (:262-267)
            if int(rep_lengths.max()) >= T:
                # the reference indexes lprobs[i, prompt_len] out of range in this case: every
                # prompt needs a leading eos (or trailing pads)
                raise IndexError("prompt without eos/pad: row prompt_len is outside the prefill")
            rows = torch.arange(BB, device=dev) * T + rep_lengths
            step_logits = flat.index_select(0, rows)
            del logits, flat

            finished = torch.zeros(BB, dtype=torch.uint8, device=dev)
            cache = decoder.get_cache(incremental_states) if hasattr(decoder, "get_cache") else None
            general = (self.sampling or self.penalties or self.penalties_src
                       or all_lprobs is not None)
            gs = self._general_state(src_tokens, BB, V, dev) if general else None
            st = None
            if (self.use_graph and all_lprobs is None and cache is not None and BB <= 64
                    and not cache.has_pads and not general):
                st = self.static_state(decoder, cache, tokens, scores, finished, step_logits)
            fused = (not general and all_lprobs is None and st is None and BB <= 128
                     and hasattr(decoder, "forward_select"))
            # Whether every row has finished is learnt one step late: the flag of a step is
            # copied to the host without waiting, the next step is launched, and only then does
            # the host wait for the flag - with work queued behind it, so the GPU never idles
            # for the host (a wait per step costs 0.15 ms: 2.5 % of a step at the OPT-6.7B
            # shape, 11 % at OPT-1.3B's).  If the flag says yes, what the extra step wrote is
            # wiped.  Rows can only finish once eos / stop tokens are allowed or forced.
            watch = _FinishWatch(finished)

            def can_end(at):
                return at >= min_len or at >= max_len - 1

            def wipe(col):
                tokens[:, col].fill_(self.pad)
                scores[:, col].fill_(0)
                if all_lprobs is not None:
                    all_lprobs[:, col].fill_(0)
            if fused:
                # the first token comes from the prefill logits; every later one is chosen inside
                # the decode step's vocabulary projection, so logits are never materialised
                step = start_step
                self._select(lib, step_logits, step, min_len, max_len, finished, tokens, scores)
                while step + 1 < max_len:
                    if can_end(step):
                        watch.post()
                    nxt = step + 1
                    decoder.forward_select(
                        tokens[:, :nxt], incremental_states, temperature=self.temperature,
                        banned=self._banned(nxt, min_len), stop=self.stop, finished=finished,
                        force_eos=nxt >= max_len - 1, eos=self.eos, tok_out=tokens[:, nxt],
                        tok_stride=tokens.stride(0), score_out=scores[:, nxt],
                        score_stride=scores.stride(0))
                    if can_end(step) and watch.all_finished():
                        wipe(nxt)
                        break
                    step = nxt
            for step in range(start_step, max_len if not fused else start_step):
                if general:
                    # masks, penalties, the step's distribution, nucleus and draw: one kernel
                    self._sample_step(lib, step_logits, step, min_len, max_len, finished, gs,
                                      tokens, scores,
                                      all_lprobs[:, step] if all_lprobs is not None else None)
                    if step > start_step and can_end(step - 1) and watch.all_finished():
                        wipe(step)  # every row had finished a step ago
                        break
                    if step + 1 >= max_len:
                        break
                    if can_end(step):
                        watch.post()
                    out = decoder(tokens[:, :step + 1], incremental_state=incremental_states)[0]
                    step_logits = out.view(BB, V)
                    continue
                if st is not None and step < max_len - 1:
                    self._graph_step(lib, st, step, min_len, max_len)
                    if step >= min_len and bool(finished.all()):
                        break
                    step_logits = st["logits"]
                    continue
                self._select(lib, step_logits, step, min_len, max_len, finished, tokens, scores)
                # rows can only finish once eos / stop tokens are allowed or forced
                if (step >= min_len or step >= max_len - 1) and bool(finished.all()):
                    break
                if step + 1 >= max_len:
                    break
                out = decoder(tokens[:, :step + 1], incremental_state=incremental_states)[0]
                step_logits = out.view(BB, V)
        finally:
            decoder.kv_cache_capacity = old_cap

        # highest cumulative score first within each sample's replicas (:325-333)
        beamscores = scores.view(bsz, beam_size, -1).cumsum(dim=-1)[:, :, -1]
        indices = beamscores.sort(dim=-1, descending=True).indices
        sorted_indices = (indices + beam_size * torch.arange(bsz, device=dev).unsqueeze(1)).view(-1)
        tokens = tokens[sorted_indices]
        scores = scores[sorted_indices]
        retval = {"tokens": tokens.view(bsz, beam_size, -1),
                  "scores": scores.view(bsz, beam_size, -1)}
        if all_lprobs is not None:
            retval["distributions"] = all_lprobs[sorted_indices].view(bsz, beam_size, -1,
                                                                      self.vocab_size)
        return retval

    # ---- general path: nucleus sampling, factual-nucleus decay, repetition penalties ----
    def _general_state(self, src_tokens, BB, V, dev):
        """Per-call buffers of the general path (:372-395)."""
        gs = {"count_tokens": None, "count_tokens_src": None}
        if self.penalties:
            gs["count_tokens"] = torch.zeros(BB, V, dtype=torch.long, device=dev)
        if self.penalties_src:
            src = src_tokens
            if self.alpha_src_penalty_end_idx > 0 and not src_tokens.shape[0] > 1:
                src = src[:, :self.alpha_src_penalty_end_idx]
            src = src.repeat_interleave(self.beam_size, 0)
            counts = torch.zeros(BB, V, dtype=torch.long, device=dev)
            counts.scatter_add_(1, src.clamp(0, V - 1), torch.ones_like(src))
            gs["count_tokens_src"] = counts
        gs["init_p"] = torch.full((BB, 1), float(self.sampling_topp), device=dev)
        gs["topp"] = gs["init_p"].clone()
        gs["toks_since_reset"] = torch.zeros(BB, 1, device=dev)
        gs["full_stop"] = torch.tensor(self.full_stop_list, device=dev)
        gs["noise"] = (torch.empty(BB, V, dtype=torch.float32, device=dev) if self.sampling
                       else None)
        return gs

    def _sample_step(self, lib, step_logits, step, min_len, max_len, finished, gs, tokens,
                     scores, lprobs_out=None):
        """One step of the general path on the device (metaseq/sequence_generator.py:272-308,
        399-441, 478-534): msa_sample_topp_f16 applies the masks and the repetition penalties,
        finds the nucleus and draws from it.  The draw consumes one Exp(1) number per row and
        token from torch's device generator (an exponential race, the way torch.multinomial
        itself draws), so ``torch.manual_seed`` fixes the samples.  ``lprobs_out`` ([BB, V] fp32
        view, any row stride) receives the step's masked, penalised log-probabilities."""
        BB, V = step_logits.shape
        banned = self._banned(step, min_len)
        ba = (ctypes.c_int32 * len(banned))(*banned)
        sa = (ctypes.c_int32 * max(1, len(self.stop)))(*self.stop)
        noise = None
        if self.sampling:
            noise = (self.noise_fn(step, BB, V) if self.noise_fn is not None
                     else gs["noise"].exponential_())
        topp_rows = gs["topp"] if (self.sampling and self.lambda_decay > 0) else None
        tok, sc = tokens[:, step], scores[:, step]
        check(lib.msa_sample_topp_f16(
            ptr(step_logits), step_logits.stride(0), BB, V, float(self.temperature), None, ba,
            len(banned), sa, len(self.stop), ptr(finished), None, int(step >= max_len - 1),
            self.eos, ptr(topp_rows), float(self.sampling_topp) if self.sampling else 0.0,
            ptr(noise), ptr(gs["count_tokens"]), ptr(gs["count_tokens_src"]),
            float(self.alpha_presence), float(self.alpha_frequency),
            float(self.alpha_presence_src), float(self.alpha_frequency_src), None,
            ptr(lprobs_out),
            lprobs_out.stride(0) if lprobs_out is not None else 0, ptr(tok), tokens.stride(0),
            ptr(sc), scores.stride(0), _capi.stream_ptr()))
        if self.sampling and self.lambda_decay > 0:
            self._update_sampling_topp(tokens[:, step], gs)

    def _update_sampling_topp(self, tok_ids, gs):
        """Factual-nucleus decay, vectorised over rows (:443-476): p restarts at its initial
        value after ".", "?" or "!" and decays by lambda_decay per further token, never below
        omega_bound."""
        hit = (tok_ids.unsqueeze(1) == gs["full_stop"].unsqueeze(0)).any(dim=1, keepdim=True)
        tsr = torch.where(hit, torch.zeros_like(gs["toks_since_reset"]),
                          gs["toks_since_reset"] + 1)
        gs["toks_since_reset"] = tsr
        decay = (tsr - 1).clamp_(min=0)
        gs["topp"] = torch.clamp(gs["init_p"] * self.lambda_decay ** decay, min=self.omega_bound)
