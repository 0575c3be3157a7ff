"""A decoder whose next-token distributions are scripted, in the spirit of the reference's
tests/utils.py:420-465: row b at history length n gets probabilities script[b][n]."""
import math

import torch


class ScriptedDecoder:
    """``script[b][n]`` = list of V probabilities predicted after n tokens of row b (missing
    entries default to uniform).  Logits are log-probabilities rounded to fp16."""

    def __init__(self, script, vocab, max_pos=64, device="cpu", dtype=torch.float32):
        self.script, self.V, self._max_pos = script, vocab, max_pos
        self.device, self.dtype = device, dtype
        self.calls = []

    def max_positions(self):
        return self._max_pos

    def _row(self, b, n):
        p = self.script.get(b, {}).get(n)
        if p is None:
            p = [1.0 / self.V] * self.V
        return [math.log(x) if x > 0 else -1e4 for x in p]

    def __call__(self, tokens, incremental_state=None, **kw):
        B, n = tokens.shape
        prefill = not incremental_state
        self.calls.append((n, prefill))
        ts = range(1, n + 1) if prefill else [n]
        out = torch.tensor([[self._row(b, t) for t in ts] for b in range(B)],
                           dtype=torch.float32).to(torch.float16).to(self.dtype).to(self.device)
        if incremental_state is not None:
            incremental_state["scripted"] = n
        return out, {"inner_states": []}

    # enough of the model surface for metaseq_amd.SequenceGenerator
    @property
    def decoder(self):
        return self

    def forward(self, tokens, **kw):
        return self(tokens, **kw)

    def max_decoder_positions(self):
        return self._max_pos

    def eval(self):
        return self

    def get_normalized_probs(self, logits, log_probs):
        return torch.log_softmax(logits.float(), -1) if log_probs else torch.softmax(
            logits.float(), -1)

    kv_cache_capacity = None


# Hand-derived cases.  Vocabulary: 0 <s>, 1 <pad>, 2 </s>, 3 <unk>, 4, 5.
L = math.log
CASES = {
    # pad has the highest probability but is never selected; eos ends the row; the loop stops.
    "eos_stops": dict(
        src=[[2, 4]], max_len_b=6, min_len=1, stop=[],
        script={0: {1: [.1, .1, .1, .1, .5, .1],      # scores the prompt token 4
                    2: [.05, .4, .05, .05, .15, .3],  # -> 5
                    3: [.1, .1, .5, .1, .1, .1]}},    # -> eos
        tokens=[[2, 4, 5, 2, 1, 1]],
        scores=[[0.0, L(.5), L(.3), L(.5), 0.0, 0.0]],
        calls=[(2, True), (3, False)]),
    # min_len blocks eos at step 3 (ties among the rest resolve to the lowest index, 0),
    # then eos at step 4.
    "min_len_blocks_eos": dict(
        src=[[2, 4]], max_len_b=6, min_len=4, stop=[],
        script={0: {1: [.1, .1, .1, .1, .5, .1],
                    2: [.05, .4, .05, .05, .15, .3],
                    3: [.1, .1, .5, .1, .1, .1],
                    4: [.1, .1, .5, .1, .1, .1]}},
        tokens=[[2, 4, 5, 0, 2, 1]],
        scores=[[0.0, L(.5), L(.3), L(.1), L(.5), 0.0]],
        calls=[(2, True), (3, False), (4, False)]),
    # nothing ever proposes eos: the last position (max_len - 1) is forced to eos.
    "forced_eos_at_max_len": dict(
        src=[[2, 5]], max_len_b=5, min_len=1, stop=[],
        script={0: {1: [.1, .1, .1, .1, .1, .5],
                    2: [.1, .1, .1, .1, .5, .1],
                    3: [.1, .1, .1, .5, .1, .1],
                    4: [.3, .1, .05, .05, .25, .25]}},
        tokens=[[2, 5, 4, 3, 2]],
        scores=[[0.0, L(.5), L(.5), L(.5), L(.05)]],
        calls=[(2, True), (3, False), (4, False)]),
    # a stop token finishes row 0 early; it then emits only eos until row 1 finishes.
    # row 1 is right-padded: its first free token comes from prefill row prompt_len = 1,
    # is written at start_step = 3 (the pad stays in the history), and its score row is
    # reset after position 1.
    "stop_token_and_padded_row": dict(
        src=[[2, 4, 5], [2, 4, 1]], max_len_b=7, min_len=1, stop=[3],
        script={0: {1: [.1, .1, .1, .1, .5, .1], 2: [.1, .1, .1, .1, .1, .5],
                    3: [.1, .1, .1, .5, .1, .1],          # -> 3 (stop) at step 3
                    4: [.5, .1, .1, .1, .1, .1],          # finished: eos, score log .1
                    5: [.1, .1, .3, .1, .2, .2]},         # finished: eos, score log .3
                1: {1: [.1, .1, .1, .1, .5, .1],
                    2: [.1, .1, .1, .1, .2, .4],          # row prompt_len=1 -> 5 at step 3
                    3: [.9, .02, .02, .02, .02, .02],     # unused (pad position row)
                    4: [.1, .1, .1, .1, .5, .1],          # -> 4 at step 4
                    5: [.1, .1, .5, .1, .1, .1]}},        # -> eos at step 5
        tokens=[[2, 4, 5, 3, 2, 2, 1], [2, 4, 1, 5, 4, 2, 1]],
        scores=[[0.0, L(.5), L(.5), L(.5), L(.1), L(.3), 0.0],
                [0.0, L(.5), 0.0, L(.4), L(.5), L(.5), 0.0]],
        calls=[(3, True), (4, False), (5, False)]),
}
