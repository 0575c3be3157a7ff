"""CPU pins for the sampling / penalty part of the oracle's generator restatement and for the
request front end's host logic.

* ``_filter_special``: the reference's own regression data
  (gpu_tests/test_hub_utils/test_filter_special_*.yml, inputs from
  ``RandomState(1234567890)`` as in gpu_tests/test_hub_utils.py:76-99), committed under
  tests/golden/filter_special/.
* nucleus mask, factual-nucleus decay, repetition penalties: hand-derived closed forms chosen so
  that an off-by-one in the cumulative mass, a missing renormalisation, a swapped
  presence/frequency coefficient or a wrong reset rule fails.
"""
import math
import os

import numpy as np
import pytest
import torch
import yaml

from metaseq_amd.hub_utils import GeneratorInterface, _IdTokenizer
from metaseq_amd.dictionary import Dictionary
from oracle import opt_oracle as O
from tests.scripted import ScriptedDecoder

GOLD = os.path.join(os.path.dirname(__file__), "golden", "filter_special")


def _gold(name):
    with open(os.path.join(GOLD, name + ".yml")) as f:
        return yaml.safe_load(f)


def test_filter_special_matches_reference_regression_data():
    tokens = [123, 453, 653, 2, 345, 453]
    prng = np.random.RandomState(1234567890)
    scores = prng.randn(len(tokens)).tolist()
    distributions = prng.randn(len(tokens), 10)
    new_tokens, new_scores, dist = GeneratorInterface._filter_special(
        pad_token_ind=1, special_token_inds=[0, 1, 2, 3], tokens=tokens, scores=scores,
        distributions=distributions)
    assert len(new_tokens) == 3 and len(new_scores) == 3
    assert new_tokens == _gold("test_filter_special_new_tokens")
    assert new_scores == pytest.approx(_gold("test_filter_special_new_scores"), abs=0, rel=1e-15)
    np.testing.assert_allclose(dist, np.array(_gold("test_filter_special_distributions")),
                               rtol=1e-15, atol=0)


def test_filter_special_pads_leading_special_and_tensor_distributions():
    # a special token at position 0 is kept, pads are skipped without ending the sequence
    toks = [2, 1, 7, 1, 8, 3, 9]
    sc = [0.0, -1.0, -2.0, -3.0, -4.0, -5.0, -6.0]
    dist = torch.arange(7 * 4, dtype=torch.float32).view(7, 4)
    t, s, d = GeneratorInterface._filter_special(1, {0, 1, 2, 3}, toks, sc, dist)
    assert t == [2, 7, 8] and s == [0.0, -2.0, -4.0]
    assert torch.equal(d, dist[[0, 2, 4]])
    t, s, d = GeneratorInterface._filter_special(1, {0, 1, 2, 3}, toks, sc, None)
    assert t == [2, 7, 8] and d is None


def test_nucleus_mask_closed_forms():
    # probabilities .5 .3 .15 .05: mass *before* a token decides (p = .8 keeps .5 and .3 since
    # the mass before .15 is exactly .8 >= p); the kept part is renormalised
    probs = torch.tensor([[.05, .5, .15, .3]])
    lp = probs.log()
    g = torch.Generator().manual_seed(0)
    _, _, trunc, sinds = O.sample_topp(lp, 0.8, g)
    assert sinds.tolist() == [[1, 3, 2, 0]]
    assert torch.allclose(trunc, torch.tensor([[.625, .375, 0., 0.]]), atol=1e-6)
    _, _, trunc, _ = O.sample_topp(lp, 0.81, g)
    assert torch.allclose(trunc, torch.tensor([[.5 / .95, .3 / .95, .15 / .95, 0.]]), atol=1e-6)
    # tiny p keeps only the arg-max; the score is the log of the *untruncated* probability
    sc, tok, trunc, _ = O.sample_topp(lp, 1e-6, g)
    assert tok.tolist() == [1] and sc.item() == pytest.approx(math.log(.5), abs=1e-6)
    # per-row p as a [rows, 1] tensor
    lp2 = torch.cat([lp, lp])
    _, _, trunc, _ = O.sample_topp(lp2, torch.tensor([[.4], [.81]]), g)
    assert torch.count_nonzero(trunc[0]) == 1 and torch.count_nonzero(trunc[1]) == 3
    # un-normalised inputs (after penalties / masks) are renormalised by the softmax
    sc, tok, trunc, _ = O.sample_topp(lp - 3.0, 1e-6, g)
    assert sc.item() == pytest.approx(math.log(.5), abs=1e-6)


def test_nucleus_sampling_frequencies():
    probs = torch.tensor([.05, .5, .15, .3])
    lp = probs.log().repeat(20000, 1)
    g = torch.Generator().manual_seed(1)
    _, tok, _, _ = O.sample_topp(lp, 0.81, g)
    freq = torch.bincount(tok, minlength=4).float() / tok.numel()
    assert freq[0] == 0
    assert torch.allclose(freq[1:], torch.tensor([.5, .15, .3]) / .95, atol=0.012)


def test_factual_nucleus_decay_closed_form():
    init_p = torch.tensor([0.9, 0.9])
    tsr = torch.zeros(2)
    full_stop = [7]
    seen = []
    for toks in ([5, 5], [5, 7], [5, 5], [5, 5], [5, 5]):
        p = O.update_sampling_topp(torch.tensor(toks), tsr, init_p, full_stop, 0.5, 0.3)
        seen.append([round(float(x), 6) for x in p])
    # row 0: counts 1,2,3,4,5 -> exponents 0,1,2,3,4 -> .9 .45 then the bound .3
    assert [s[0] for s in seen] == [0.9, 0.45, 0.3, 0.3, 0.3]
    # row 1: reset by the full stop at the 2nd token: counts 1,0,1,2,3 -> exponents 0,0,0,1,2
    assert [s[1] for s in seen] == [0.9, 0.9, 0.9, 0.45, 0.3]


def test_repetition_penalties_closed_form():
    lp = torch.zeros(1, 4)
    c = torch.tensor([[0, 1, 3, 0]])
    cs = torch.tensor([[2, 0, 1, 0]])
    out = O.apply_repetition_penalties(lp, c, cs, alpha_presence=0.5, alpha_frequency=0.1,
                                       alpha_presence_src=0.25, alpha_frequency_src=1.0)
    want = torch.tensor([[-(0.25 + 2.0), -(0.5 + 0.1), -(0.5 + 0.3) - (0.25 + 1.0), 0.0]])
    assert torch.allclose(out, want, atol=1e-6)
    # one coefficient alone switches its pair on; zero coefficients leave lprobs untouched
    assert torch.equal(O.apply_repetition_penalties(lp, c, cs), lp)
    out = O.apply_repetition_penalties(lp, c, cs, alpha_frequency=0.1)
    assert torch.allclose(out, torch.tensor([[0.0, -0.1, -0.3, 0.0]]), atol=1e-6)


def test_oracle_generate_penalties_change_the_greedy_path():
    """Scripted decoder that always prefers token 4: a presence penalty on generated tokens
    makes the second pick the runner-up, and a prompt penalty moves the first pick."""
    row = [.02, .02, .02, .02, .5, .3, .12]
    script = {0: {n: row for n in range(1, 8)}}
    src = torch.tensor([[2, 6]])
    dec = ScriptedDecoder(script, 7)
    base = O.generate(dec, src, max_len_b=5, min_len=4)["tokens"][0, 0].tolist()
    assert base == [2, 6, 4, 4, 2]
    dec = ScriptedDecoder(script, 7)
    pen = O.generate(dec, src, max_len_b=5, min_len=4, alpha_presence=1.0)
    assert pen["tokens"][0, 0].tolist() == [2, 6, 4, 5, 2]
    # the recorded score of the penalised pick is the penalised log-probability
    assert pen["scores"][0, 0, 3].item() == pytest.approx(math.log(.3), abs=2e-3)
    row2 = [.02, .02, .02, .02, .3, .12, .5]
    dec = ScriptedDecoder({0: {n: row2 for n in range(1, 8)}}, 7)
    srcpen = O.generate(dec, src, max_len_b=5, min_len=4, alpha_presence_src=2.0)
    assert srcpen["tokens"][0, 0].tolist() == [2, 6, 4, 4, 2]   # 6 is in the prompt


def test_build_batch_prepends_eos_and_right_pads():
    gi = GeneratorInterface(model=None, tgt_dict=Dictionary(50), max_positions=64)
    b = gi.build_batch([[5, 6, 7], [9], []])
    assert b["net_input"]["src_tokens"].tolist() == [[2, 5, 6, 7], [2, 9, 1, 1], [2, 1, 1, 1]]
    assert b["net_input"]["src_lengths"].tolist() == [4, 2, 1]


def test_record_assembly_echo_and_cut():
    gi = GeneratorInterface(model=None, tgt_dict=Dictionary(50), max_positions=64)
    # row: eos, prompt 5 6, pad (shorter prompt in a padded batch), generated 7 8, eos, pad
    tokens = [2, 5, 6, 1, 7, 8, 2, 1]
    scores = [0.0, -.1, -.2, 0.0, -.3, -.4, -.5, 0.0]
    dist = torch.arange(8 * 50, dtype=torch.float32).view(8, 50)
    r = gi._record(list(tokens), list(scores), dist, prompt_len=2, max_tokens=1, echo=False,
                   logprobs=2)
    assert r["tokens"] == ["7"] and r["token_scores"] == [-.3] and r["text"] == "7"
    assert r["text_offset"] == [0]
    assert r["top_logprobs"] == [{"49": float(dist[4, 49]), "48": float(dist[4, 48])}]
    r = gi._record(list(tokens), list(scores), None, prompt_len=2, max_tokens=5, echo=True,
                   logprobs=0)
    assert r["tokens"] == ["2", "5", "6", "7", "8"]
    assert r["token_scores"] == [None, -.1, -.2, -.3, -.4]
    assert r["text"] == "5 6 7 8" and r["text_offset"] == [0, 2, 4, 6]
    assert r["top_logprobs"] is None


def test_id_tokenizer_round_trip():
    tk = _IdTokenizer()
    text = tk.decode([12, 7, 50271])
    enc = tk.encode(text)
    assert enc.ids == [12, 7, 50271] and enc.offsets == [(0, 2), (3, 4), (5, 10)]
    assert tk.encode("").ids == []


def test_dictionary_resolves_symbols_from_a_table_or_a_tokenizer():
    class Tok:
        def token_to_id(self, s):
            return {".": 13, "?": 30}.get(s)
    plain = Dictionary(100)
    assert plain.index(".") == plain.unk() == 3 and not plain.resolves(".")
    table = Dictionary(100, symbols={".": 4, "!": 6})
    assert (table.index("."), table.index("!"), table.index("?")) == (4, 6, 3)
    tok = Dictionary(100, tokenizer=Tok())
    assert (tok.index("."), tok.index("?"), tok.index("!")) == (13, 30, 3)
    assert tok.resolves("?") and not tok.resolves("!")


def test_factual_nucleus_needs_resolvable_full_stops():
    """With a dictionary that maps ".", "?" and "!" to <unk> the decayed nucleus would never be
    reset (the reference resets on dictionary.index(...), sequence_generator.py:116, 443-476):
    the generator refuses that combination instead of decaying silently."""
    from metaseq_amd import SequenceGenerator
    dec = ScriptedDecoder({0: {1: [1.0] + [0.0] * 11}}, 12)
    with pytest.raises(ValueError, match="lambda_decay"):
        SequenceGenerator([dec], Dictionary(12), topp=0.9, lambda_decay=0.8)
    gen = SequenceGenerator([dec], Dictionary(12, symbols={".": 7, "?": 8, "!": 9}), topp=0.9,
                            lambda_decay=0.8)
    assert gen.full_stop_list == [7, 8, 9]
    SequenceGenerator([dec], Dictionary(12), topp=0.9)  # no decay: nothing to resolve


def test_exponential_race_draws_from_the_truncated_distribution():
    """sample_topp with noise: the arg-max of probability / Exp(1) noise over the nucleus picks
    every id with its renormalised nucleus probability (frequencies over 20 000 draws), never an
    id outside the nucleus, and scores it with its untruncated log-probability."""
    probs = torch.tensor([0.05, 0.4, 0.1, 0.25, 0.2])
    n = 20000
    lprobs = probs.log().unsqueeze(0).repeat(n, 1)
    noise = torch.empty(n, 5).exponential_(generator=torch.Generator().manual_seed(5))
    sc, tok, _, _ = O.sample_topp(lprobs, 0.7, noise=noise)   # nucleus: 0.4, 0.25, 0.2
    assert set(tok.tolist()) == {1, 3, 4}
    freq = torch.bincount(tok, minlength=5).float() / n
    assert torch.allclose(freq, torch.tensor([0, 0.4, 0, 0.25, 0.2]) / 0.85, atol=0.012)
    assert torch.allclose(sc, probs[tok].log(), atol=1e-6)
