"""Known-answer tests of the oracle's greedy loop with scripted distributions; expected
tokens, scores and decoder-call sequences were derived by hand from the reference's loop
(metaseq/sequence_generator.py:223-323)."""
import pytest
import torch

from oracle.opt_oracle import greedy_generate
from tests.scripted import CASES, ScriptedDecoder


@pytest.mark.parametrize("name", sorted(CASES))
def test_scripted_known_answers(name):
    c = CASES[name]
    dec = ScriptedDecoder(c["script"], vocab=6)
    out = greedy_generate(dec, torch.tensor(c["src"]), max_len_b=c["max_len_b"],
                          min_len=c["min_len"], stop=c["stop"])
    assert out["tokens"][:, 0].tolist() == c["tokens"]
    got = out["scores"][:, 0]
    want = torch.tensor(c["scores"])
    assert torch.allclose(got, want, atol=2e-3), (got, want)
    assert dec.calls == c["calls"]


def test_max_len_is_capped_by_model_positions():
    dec = ScriptedDecoder({}, vocab=6, max_pos=4)
    out = greedy_generate(dec, torch.tensor([[2, 4]]), max_len_b=50, min_len=1)
    assert out["tokens"].shape == (1, 1, 4)
    assert out["tokens"][0, 0, -1].item() == 2  # forced eos at the cap
