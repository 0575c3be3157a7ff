"""The generator's general path (nucleus sampling, factual-nucleus decay, repetition penalties)
and the request front end on the GPU.

Parity for sampling is exact, not statistical: with a scripted decoder both sides see identical
log-probabilities, and the oracle (run on the same device) is handed the very Exp(1) numbers the
product's sampling kernel draws with, so the tokens must agree exactly - with ``need_logprobs``
too, where the same kernel also writes every step's distribution.  The draw rule itself is
pinned on the CPU (frequencies and nucleus membership).
"""
import math

import pytest
import torch

from metaseq_amd import (Dictionary, GeneratorInterface, SequenceGenerator,
                         TransformerLanguageModel, random_prompts, random_state_dict)
from oracle import opt_oracle as O
from tests.common import make_oracle, tiny_cfg
from tests.scripted import ScriptedDecoder

pytestmark = pytest.mark.gpu
DEV = "cuda"
V = 12
# ids the test dictionary gives ".", "?" and "!": ordinary tokens of the scripted vocabulary, so
# the factual-nucleus resets really fire
FULL_STOPS = {".": 7, "?": 8, "!": 9}


def _script(B, seed):
    g = torch.Generator().manual_seed(seed)
    script = {}
    for b in range(B):
        script[b] = {}
        for n in range(1, 24):
            p = torch.rand(V, generator=g) ** 3 + 1e-3
            script[b][n] = (p / p.sum()).tolist()
    return script


def _both(kw, B=3, seed=11, beam=1, max_len_b=16, min_len=6, src=None):
    script = _script(B * beam, seed)
    if src is None:
        src = torch.tensor([[2, 5, 7, 9], [2, 6, 1, 1], [2, 4, 8, 1]][:B])
    dec = ScriptedDecoder(script, V, device=DEV, dtype=torch.float16)
    gen = SequenceGenerator([dec], Dictionary(V, symbols=FULL_STOPS), beam_size=beam,
                            max_len_b=max_len_b, min_len=min_len, **kw)
    torch.manual_seed(1234)
    got = gen.generate([dec], {"net_input": {"src_tokens": src.to(DEV)}})
    dec2 = ScriptedDecoder(script, V, device=DEV, dtype=torch.float16)
    torch.manual_seed(1234)
    # the kernel draws by an exponential race over token ids, one Exp(1) number per row and id
    # and step from the device generator; the oracle is handed the same numbers
    noise_fn = lambda shape: torch.empty(shape, dtype=torch.float32, device=DEV).exponential_()
    want = O.generate(dec2, src.to(DEV), max_len_b=max_len_b, min_len=min_len, beam_size=beam,
                      full_stop_list=tuple(FULL_STOPS.values()), noise_fn=noise_fn, **kw)
    return got, want


@pytest.mark.parametrize("kw", [
    dict(topp=0.9),
    dict(topp=0.5, temperature=0.7),
    dict(topp=0.95, stop=[10]),
    dict(topp=0.9, lambda_decay=0.8, omega_bound=0.2),
    dict(topp=0.9, alpha_presence=0.7, alpha_frequency=0.2),
    dict(alpha_presence=1.5, alpha_frequency=0.5),                    # greedy with penalties
    dict(alpha_presence_src=1.0, alpha_frequency_src=0.3),
    dict(topp=0.8, alpha_presence=0.5, alpha_presence_src=0.5, alpha_frequency_src=0.1,
         need_logprobs=True),
    dict(need_logprobs=True, temperature=0.8, stop=[10]),            # greedy, distributions kept
], ids=lambda k: ",".join("%s=%s" % kv for kv in k.items()))
def test_general_path_matches_oracle_bit_for_bit(kw):
    got, want = _both(kw)
    assert torch.equal(got["tokens"], want["tokens"]), (got["tokens"], want["tokens"])
    n0 = 4
    # scores and distributions: the kernels' fp32 summation order differs from the tensor ops'
    assert torch.allclose(got["scores"], want["scores"], atol=2e-5)
    if kw.get("need_logprobs"):
        gd, wd = got["distributions"], want["distributions"]
        assert gd.shape == wd.shape
        assert torch.equal(torch.isinf(gd), torch.isinf(wd)), "masked ids differ"
        ok = torch.isfinite(wd)
        assert torch.allclose(gd[ok], wd[ok], atol=2e-5)
        assert bool(torch.isfinite(gd[:, :, n0:]).any())
    # sampling really happened: some pick is not the arg-max of its distribution
    if kw.get("topp", 0) >= 0.8:
        greedy, _ = _both({k: v for k, v in kw.items() if k != "topp"})
        assert not torch.equal(greedy["tokens"], got["tokens"])


def test_sampling_with_replicas_sorted_by_score():
    got, want = _both(dict(topp=0.9), B=2, beam=3)
    assert torch.equal(got["tokens"], want["tokens"])
    assert torch.allclose(got["scores"], want["scores"], atol=2e-5)
    tot = got["scores"].sum(-1)
    assert bool((tot[:, :-1] >= tot[:, 1:]).all())
    assert not torch.equal(got["tokens"][:, 0], got["tokens"][:, 1])


def test_src_penalty_end_index_single_prompt():
    src = torch.tensor([[2, 5, 7, 9, 5]])
    kw = dict(alpha_presence_src=2.0, alpha_src_penalty_end_idx=3)
    got, want = _both(kw, B=1, src=src, max_len_b=14, min_len=8)
    assert torch.equal(got["tokens"], want["tokens"])
    # token 9 (outside the first 3 prompt tokens) is not penalised, so the runs differ
    got2, _ = _both(dict(alpha_presence_src=2.0), B=1, src=src, max_len_b=14, min_len=8)
    assert not torch.equal(got["scores"], got2["scores"])


def test_samples_stay_inside_the_nucleus_on_a_real_model():
    cfg = tiny_cfg(layers=2, dim=128, heads=2, vocab=64, max_pos=48)
    sd = random_state_dict(cfg, seed=5, dtype=torch.float16)
    model = TransformerLanguageModel.build_model(cfg, sd, device=DEV)
    src = random_prompts(cfg, 4, 6, seed=3).to(DEV)
    gen = SequenceGenerator([model], Dictionary(cfg.vocab_size), max_len_b=24, min_len=23,
                            topp=0.6, need_logprobs=True)
    torch.manual_seed(7)
    out = gen.generate([model], {"net_input": {"src_tokens": src}})
    toks, dist = out["tokens"][:, 0], out["distributions"][:, 0]
    n0 = src.shape[1]
    for t in range(n0, 23):
        p = torch.softmax(dist[:, t], -1)
        sp, si = p.sort(-1, descending=True)
        before = sp.cumsum(-1) - sp
        rank = (si == toks[:, t].unsqueeze(1)).float().argmax(-1)
        assert bool((before.gather(1, rank.unsqueeze(1)) < 0.6).all()), t
        chosen = dist[:, t].gather(1, toks[:, t].unsqueeze(1)).squeeze(1)
        assert torch.allclose(out["scores"][:, 0, t], torch.log_softmax(dist[:, t], -1).gather(
            1, toks[:, t].unsqueeze(1)).squeeze(1), atol=1e-5)
        assert bool(torch.isfinite(chosen).all())
    # same seed, same tokens; another seed, other tokens
    torch.manual_seed(7)
    again = gen.generate([model], {"net_input": {"src_tokens": src}})
    assert torch.equal(again["tokens"], out["tokens"])
    torch.manual_seed(8)
    other = gen.generate([model], {"net_input": {"src_tokens": src}})
    assert not torch.equal(other["tokens"], out["tokens"])


def _interface(vocab=64, max_pos=48):
    cfg = tiny_cfg(layers=2, dim=128, heads=2, vocab=vocab, max_pos=max_pos)
    sd = random_state_dict(cfg, seed=21, dtype=torch.float16)
    model = TransformerLanguageModel.build_model(cfg, sd, device=DEV)
    return GeneratorInterface(model, Dictionary(cfg.vocab_size)), model, cfg, sd


def test_interface_greedy_matches_oracle_generation_on_ragged_prompts():
    gi, model, cfg, sd = _interface()
    prompts = [[5, 9, 33, 12, 7], [40, 41], [8, 8, 8]]
    res = gi.generate(prompts, max_tokens=[6, 4, 6], min_tokens=[6, 4, 6], temperature=1.0,
                      top_p=-1.0, n=1, echo=False)
    src = gi.build_batch(prompts)["net_input"]["src_tokens"]
    oracle = make_oracle(cfg, sd, torch.float16)
    want = O.generate(oracle, src, max_len_b=min(48, 6 + 6), min_len=6 + 6)
    for i, p in enumerate(prompts):
        row = want["tokens"][i, 0].tolist()
        t, s, _ = GeneratorInterface._filter_special(1, {0, 1, 2, 3}, row,
                                                     want["scores"][i, 0].tolist(), None)
        cut = t[len(p) + 1:][:[6, 4, 6][i]]
        rec = res[i][0]
        assert rec["tokens"] == [str(x) for x in cut], (i, rec["tokens"], cut)
        assert rec["text"] == " ".join(str(x) for x in cut)
        assert rec["top_logprobs"] is None
        assert len(rec["token_scores"]) == len(cut)
        assert all(abs(a - b) < 5e-2 for a, b in
                   zip(rec["token_scores"], s[len(p) + 1:][:[6, 4, 6][i]]))


def test_interface_echo_scores_the_prompt_and_logprobs_hold_the_choice():
    gi, model, cfg, sd = _interface()
    prompt = [5, 9, 33, 12, 7, 20]
    [[rec]] = gi.generate([prompt], max_tokens=[0], min_tokens=[0], echo=True, logprobs=3)
    # echo with max_tokens 0: the eos-prefixed prompt and one forced end-of-sentence, which
    # _filter_special removes; the first score is withheld
    assert rec["tokens"] == ["2"] + [str(t) for t in prompt]
    assert rec["token_scores"][0] is None and len(rec["token_scores"]) == len(prompt) + 1
    oracle = make_oracle(cfg, sd, torch.float16)
    logits = oracle(torch.tensor([[2] + prompt]))[0].float()
    lp = torch.log_softmax(logits, -1)[0]
    want = [float(lp[i, prompt[i]]) for i in range(len(prompt))]
    assert all(abs(a - b) < 5e-2 for a, b in zip(rec["token_scores"][1:], want))
    assert rec["top_logprobs"][0] is None and len(rec["top_logprobs"]) == len(prompt) + 1
    for i in range(1, len(prompt) + 1):
        top = rec["top_logprobs"][i]
        assert len(top) == 3
        best = max(top.values())
        assert abs(best - float(lp[i - 1].max())) < 5e-2
    # greedy continuation: the chosen token is the top entry of its own distribution
    [[rec]] = gi.generate([prompt], max_tokens=[5], min_tokens=[5], logprobs=2)
    for tok, sc, top in zip(rec["tokens"], rec["token_scores"], rec["top_logprobs"]):
        assert tok in top and abs(top[tok] - sc) < 1e-5 and top[tok] == max(top.values())


def test_interface_sampling_n_best_of_and_seed():
    gi, model, cfg, sd = _interface()
    prompts = [[5, 9, 33], [40, 41, 42]]
    kw = dict(max_tokens=[8, 8], min_tokens=[7, 7], top_p=0.9, n=2, best_of=4, seed=3)
    a = gi.generate(prompts, **kw)
    b = gi.generate(prompts, **kw)
    assert a == b
    assert len(a) == 2 and all(len(beams) == 2 for beams in a)
    for beams in a:
        # replicas come best cumulative score first; a sampled <s> or <unk> cuts a record short,
        # like any special token, so only uncut records can be compared by their score sums
        assert all(len(r["tokens"]) <= 8 for r in beams)
        if all(len(r["token_scores"]) == 7 for r in beams):
            assert sum(beams[0]["token_scores"]) >= sum(beams[1]["token_scores"]) - 1e-6
    c = gi.generate(prompts, **dict(kw, seed=4))
    assert c != a
    # temperature 0 means greedy whatever top_p says
    g0 = gi.generate(prompts, max_tokens=[4, 4], min_tokens=[4, 4], temperature=0, top_p=0.9)
    g1 = gi.generate(prompts, max_tokens=[4, 4], min_tokens=[4, 4])
    assert g0 == g1
    with pytest.raises(ValueError):
        gi.generate(prompts, temperature=-1)


def test_fully_masked_step_does_not_reach_multinomial_with_nan():
    """min_len == max_len leaves no selectable token at the last step (eos is blocked and
    everything else is forced off).  The reference's sampler raises there; the product gives
    the row what its greedy branch would: token 0 with score -inf."""
    script = _script(2, 5)
    dec = ScriptedDecoder(script, V, device=DEV, dtype=torch.float16)
    gen = SequenceGenerator([dec], Dictionary(V), max_len_b=8, min_len=8, topp=0.9)
    torch.manual_seed(0)
    out = gen.generate([dec], {"net_input": {"src_tokens": torch.tensor(
        [[2, 5, 7], [2, 6, 4]], device=DEV)}})
    torch.cuda.synchronize()
    assert out["tokens"][:, 0, 7].tolist() == [0, 0]
    assert bool(torch.isinf(out["scores"][:, 0, 7]).all())
    assert bool(torch.isfinite(out["scores"][:, 0, :7]).all())


def test_batching_service_over_the_interface_returns_what_direct_calls_return():
    from metaseq_amd.service import BatchingService
    gi, model, cfg, sd = _interface()
    prompts = [[5, 9, 33, 12, 7], [40, 41], [8, 8, 8]]
    svc = BatchingService(gi, max_seq_len=48, timeout_ms=5)
    rets = [svc.submit(p, max_tokens=5, min_tokens=4, temperature=1.0, top_p=-1.0, n=1)
            for p in prompts]
    assert svc.step() == 3          # one padded batch for the three prompts
    direct = gi.generate(prompts, max_tokens=[5] * 3, min_tokens=[4] * 3)
    # the service hands prompts over cheapest first; every caller still gets its own row
    for p, r, want in zip(prompts, rets, direct):
        uid, got = r.get_nowait()
        assert got[0]["tokens"] == want[0]["tokens"], p


def test_continuous_batcher_rows_equal_single_request_generation():
    """Requests that join and leave a running batch of slots get exactly what a generation of
    their own would give them: with at most 16 rows every row runs through the same kernels
    with the same summation order whatever its neighbours are, so tokens and scores are equal to
    the last bit.  More requests than slots, different prompt lengths, minimum and maximum
    lengths, echo."""
    from metaseq_amd.service import ContinuousBatcher
    gi, model, cfg, sd = _interface()
    specs = [dict(prompt=[5, 9, 33, 12, 7], max_tokens=9),
             dict(prompt=[40], max_tokens=3),
             dict(prompt=[8, 8, 8, 21, 22, 23, 24, 25, 26, 27, 28], min_tokens=5, max_tokens=12),
             dict(prompt=[17, 4], max_tokens=1),
             dict(prompt=[30, 31, 32], min_tokens=2, max_tokens=7, echo=True),
             dict(prompt=[11], max_tokens=14),
             dict(prompt=[45, 46, 47, 48], max_tokens=6)]
    cb = ContinuousBatcher(gi, slots=3, capacity=40)
    replies = [cb.submit(s["prompt"], **{k: v for k, v in s.items() if k != "prompt"})
               for s in specs]
    n = 0
    while cb.step():
        n += 1
        assert n < 200
    assert cb.steps > 0 and cb.rows_stepped > cb.steps      # rows shared decode steps
    for s, r in zip(specs, replies):
        _, got = r.get_nowait()
        assert not isinstance(got, Exception), got
        want = gi.generate([s["prompt"]], max_tokens=[s["max_tokens"]],
                           min_tokens=[s.get("min_tokens", 0)], echo=s.get("echo", False))
        assert got[0]["tokens"] == want[0][0]["tokens"], s
        assert got[0]["token_scores"] == want[0][0]["token_scores"], s
        assert got[0]["text"] == want[0][0]["text"]
    # every slot is free again and the cache holds no active row
    assert cb.cache.lens.tolist() == [-1, -1, -1]


def _noise_for(prompt, replica, position, vocab):
    """Exp(1) numbers that depend only on the request's prompt, the replica and the position of
    the token being drawn, so that two engines can be handed the same ones."""
    g = torch.Generator(device=DEV).manual_seed(7919 * sum(prompt) + 101 * replica + position)
    return torch.empty(vocab, dtype=torch.float32, device=DEV).exponential_(generator=g)


def test_continuous_batcher_sampled_rows_equal_single_request_generation():
    """Sampled requests (each with its own temperature and top-p), greedy requests at another
    temperature, plainly greedy ones and requests with several replicas share the slots of one
    running batch.  Given the same noise per (request, replica, position), every request gets
    the tokens and scores of a generation of its own: its rows run through the same kernels on
    the same logits, whatever their neighbours are and however they are chosen."""
    from metaseq_amd.service import ContinuousBatcher
    gi, model, cfg, sd = _interface()
    specs = [dict(prompt=[5, 9, 33, 12, 7], max_tokens=9, temperature=0.7, top_p=0.9),
             dict(prompt=[40], max_tokens=5),
             dict(prompt=[8, 8, 8, 21, 22, 23, 24, 25], min_tokens=5, max_tokens=12, top_p=0.5),
             dict(prompt=[17, 4], max_tokens=6, temperature=0.5),
             dict(prompt=[30, 31, 32], min_tokens=2, max_tokens=7, temperature=1.2, top_p=0.95,
                  n=2, best_of=3),
             dict(prompt=[11], max_tokens=10, temperature=0, top_p=0.9),
             dict(prompt=[45, 46, 47, 48], max_tokens=6, top_p=1.0, echo=True)]
    cb = ContinuousBatcher(gi, slots=5, capacity=40,
                           noise_fn=lambda req, j, pos, V: _noise_for(req.prompt, j, pos, V))
    replies = [cb.submit(s["prompt"], **{k: v for k, v in s.items() if k != "prompt"})
               for s in specs]
    n = 0
    while cb.step():
        n += 1
        assert n < 300
    assert cb.rows_stepped > cb.steps > 0
    for s, r in zip(specs, replies):
        _, got = r.get_nowait()
        assert not isinstance(got, Exception), got
        prompt = s["prompt"]
        gi.noise_fn = lambda step, BB, V: torch.stack(
            [_noise_for(prompt, j, step, V) for j in range(BB)])
        want = gi.generate([prompt], max_tokens=[s["max_tokens"]],
                           min_tokens=[s.get("min_tokens", 0)], echo=s.get("echo", False),
                           temperature=s.get("temperature", 1.0), top_p=s.get("top_p", -1.0),
                           n=s.get("n", 1), best_of=s.get("best_of"))[0]
        gi.noise_fn = None
        assert len(got) == len(want) == s.get("n", 1)
        for g_rec, w_rec in zip(got, want):
            assert g_rec["tokens"] == w_rec["tokens"], (s, g_rec["tokens"], w_rec["tokens"])
            assert g_rec["token_scores"] == w_rec["token_scores"], s
        if s is specs[0]:
            # sampling happened: the continuation is not the request's greedy one
            greedy = gi.generate([prompt], max_tokens=[9], min_tokens=[0])[0][0]
            assert greedy["tokens"] != got[0]["tokens"]
    assert cb.cache.lens.tolist() == [-1] * 5


def test_continuous_batcher_penalties_decaying_nucleus_and_logprobs_equal_single_requests():
    """Requests with repetition penalties (generated and prompt tokens, the prompt counts cut at
    alpha_src_penalty_end_idx), with the factual-nucleus decay, with ``logprobs`` (with and
    without ``echo``) and plain ones share the slots of one running batch.  Given the same noise
    per (request, replica, position), each gets the tokens, the scores and the per-position
    alternatives of a generation of its own through SequenceGenerator's general path."""
    from metaseq_amd.service import ContinuousBatcher
    cfg = tiny_cfg(layers=2, dim=128, heads=2, vocab=64, max_pos=48)
    sd = random_state_dict(cfg, seed=21, dtype=torch.float16)
    model = TransformerLanguageModel.build_model(cfg, sd, device=DEV)
    stops = {".": 13, "?": 29, "!": 41}
    gi = GeneratorInterface(model, Dictionary(cfg.vocab_size, symbols=stops))
    specs = [dict(prompt=[5, 9, 5, 5, 7], max_tokens=12, alpha_presence=0.8, alpha_frequency=0.6),
             dict(prompt=[8, 8, 8, 21], max_tokens=14, temperature=0.9, top_p=0.9,
                  lambda_decay=0.6, omega_bound=0.2),
             dict(prompt=[40, 41], max_tokens=6, logprobs=3),
             dict(prompt=[17, 4, 17, 17], max_tokens=9, alpha_presence_src=0.7,
                  alpha_frequency_src=0.5, alpha_src_penalty_end_idx=3, top_p=0.7, logprobs=2,
                  echo=True),
             dict(prompt=[30, 31, 32], max_tokens=7),
             dict(prompt=[33, 13, 11], max_tokens=12, min_tokens=3, top_p=0.8, lambda_decay=0.5,
                  alpha_frequency=0.4, n=2, best_of=2, logprobs=1)]
    cb = ContinuousBatcher(gi, slots=4, capacity=40,
                           noise_fn=lambda req, j, pos, V: _noise_for(req.prompt, j, pos, V))
    replies = [cb.submit(s["prompt"], **{k: v for k, v in s.items() if k != "prompt"})
               for s in specs]
    n = 0
    while cb.step():
        n += 1
        assert n < 300
    assert cb.rows_stepped > cb.steps > 0
    extras = ("lambda_decay", "omega_bound", "alpha_presence", "alpha_frequency",
              "alpha_presence_src", "alpha_frequency_src", "alpha_src_penalty_end_idx", "logprobs")
    for s, r in zip(specs, replies):
        _, got = r.get_nowait()
        assert not isinstance(got, Exception), (s, got)
        prompt = s["prompt"]
        gi.noise_fn = lambda step, BB, V: torch.stack(
            [_noise_for(prompt, j, step, V) for j in range(BB)])
        want = gi.generate([prompt], max_tokens=[s["max_tokens"]],
                           min_tokens=[s.get("min_tokens", 0)], echo=s.get("echo", False),
                           temperature=s.get("temperature", 1.0), top_p=s.get("top_p", -1.0),
                           n=s.get("n", 1), best_of=s.get("best_of"),
                           **{k: s[k] for k in extras if k in s})[0]
        gi.noise_fn = None
        assert len(got) == len(want) == s.get("n", 1)
        for g_rec, w_rec in zip(got, want):
            assert g_rec["tokens"] == w_rec["tokens"], (s, g_rec["tokens"], w_rec["tokens"])
            assert g_rec["token_scores"] == w_rec["token_scores"], s
            if not s.get("logprobs"):
                assert g_rec["top_logprobs"] is None and w_rec["top_logprobs"] is None
                continue
            assert len(g_rec["top_logprobs"]) == len(w_rec["top_logprobs"])
            for pos, (g_top, w_top) in enumerate(zip(g_rec["top_logprobs"], w_rec["top_logprobs"])):
                if w_top is None:
                    assert g_top is None
                    continue
                # the same values; the same ids wherever a value is not tied with the next one
                # (the two sides rank ties by different routines)
                gv, wv = sorted(g_top.values()), sorted(w_top.values())
                assert gv == wv, (s, pos, g_top, w_top)
                if len(set(wv)) == len(wv) and len(w_top) == s["logprobs"]:
                    assert g_top == w_top, (s, pos, g_top, w_top)
        if s is specs[0]:
            # the penalties acted: the continuation is not the request's unpenalised one
            base = gi.generate([prompt], max_tokens=[12], min_tokens=[0])[0][0]
            assert base["tokens"] != got[0]["tokens"]
    assert cb.cache.lens.tolist() == [-1] * 4


@pytest.mark.parametrize("int8", [False, True])
def test_continuous_batcher_with_more_than_128_slots(int8):
    """150 slots: the running batch leaves the packed path (row-major activations through the
    tile kernels with per-row lengths; int8 weights: chunks of at most 128 rows through the
    packed path).  Requests of different lengths, some sampled, join and leave; each gets what
    a generation of its own gives - the logits now come from other kernels than a single
    request's, so a near-tie may be decided the other way in a few requests, and scores agree
    to the kernels' tolerance rather than to the bit."""
    from metaseq_amd.service import ContinuousBatcher
    cfg = tiny_cfg(layers=2, dim=128, heads=2, vocab=64, max_pos=48)
    sd = random_state_dict(cfg, seed=21, dtype=torch.float16)
    model = TransformerLanguageModel.build_model(cfg, sd, device=DEV)
    if int8:
        model.decoder.quantize_int8_()
    gi = GeneratorInterface(model, Dictionary(cfg.vocab_size))
    g = torch.Generator().manual_seed(5)
    specs = []
    for i in range(190):
        n = int(torch.randint(1, 9, (1,), generator=g))
        spec = dict(prompt=torch.randint(4, 64, (n,), generator=g).tolist(),
                    max_tokens=int(torch.randint(6, 20, (1,), generator=g)))
        if i % 7 == 0:
            spec.update(temperature=0.8, top_p=0.9)
        if i % 11 == 0:
            spec.update(min_tokens=min(3, spec["max_tokens"]))
        specs.append(spec)
    cb = ContinuousBatcher(gi, slots=150, capacity=32,
                           noise_fn=lambda req, j, pos, V: _noise_for(req.prompt, j, pos, V))
    replies = [cb.submit(s["prompt"], **{k: v for k, v in s.items() if k != "prompt"})
               for s in specs]
    n = widest = 0
    while cb.step():
        n += 1
        assert n < 400
        widest = max(widest, int((cb.cache.lens >= 0).sum()))
    assert widest > 128      # steps really ran with more rows than the packed path takes
    same = 0
    for s, r in zip(specs, replies):
        _, got = r.get_nowait()
        assert not isinstance(got, Exception), (s, got)
        prompt = s["prompt"]
        gi.noise_fn = lambda step, BB, V: torch.stack(
            [_noise_for(prompt, j, step, V) for j in range(BB)])
        want = gi.generate([prompt], max_tokens=[s["max_tokens"]],
                           min_tokens=[s.get("min_tokens", 0)],
                           temperature=s.get("temperature", 1.0), top_p=s.get("top_p", -1.0))[0]
        gi.noise_fn = None
        if got[0]["tokens"] == want[0]["tokens"]:
            same += 1
            assert all(abs(a - b) < 2e-2 for a, b in zip(got[0]["token_scores"],
                                                         want[0]["token_scores"])), s
    print("more than 128 slots, int8=%s: %d / %d requests identical to their own generation"
          % (int8, same, len(specs)), flush=True)
    assert same >= len(specs) - 6
    assert cb.cache.lens.tolist() == [-1] * 150


def test_continuous_batcher_with_shared_prefills():
    """prefill_batch / prefill_wait: waiting requests share prefills (other tile shapes than a
    prompt's own prefill), so a near-tie may be decided the other way in a few requests;
    all others get the tokens of a generation of their own, with scores to the kernels'
    tolerance."""
    from metaseq_amd.service import ContinuousBatcher
    gi, model, cfg, sd = _interface()
    g = torch.Generator().manual_seed(9)
    specs = []
    for i in range(60):
        n = int(torch.randint(1, 12, (1,), generator=g))
        spec = dict(prompt=torch.randint(4, 64, (n,), generator=g).tolist(),
                    max_tokens=int(torch.randint(3, 18, (1,), generator=g)))
        if i % 3 == 0:
            spec.update(temperature=0.8, top_p=0.9)
        if i % 5 == 0:
            spec.update(n=2, best_of=2, top_p=0.7)
        specs.append(spec)
    cb = ContinuousBatcher(gi, slots=12, capacity=32, prefill_batch=5, prefill_wait=3,
                           noise_fn=lambda req, j, pos, V: _noise_for(req.prompt, j, pos, V))
    shared = []
    inner = cb.decoder.admit_slots
    cb.decoder.admit_slots = lambda cache, reqs, **kw: (shared.append(len(reqs)),
                                                        inner(cache, reqs, **kw))[1]
    try:
        replies = [cb.submit(s["prompt"], **{k: v for k, v in s.items() if k != "prompt"})
                   for s in specs]
        n = 0
        while cb.step():
            n += 1
            assert n < 600
    finally:
        del cb.decoder.admit_slots
    assert shared and max(shared) > 1, shared
    same = 0
    for s, r in zip(specs, replies):
        _, got = r.get_nowait()
        assert not isinstance(got, Exception), (s, got)
        prompt = s["prompt"]
        gi.noise_fn = lambda step, BB, V: torch.stack(
            [_noise_for(prompt, j, step, V) for j in range(BB)])
        want = gi.generate([prompt], max_tokens=[s["max_tokens"]], min_tokens=[0],
                           temperature=s.get("temperature", 1.0), top_p=s.get("top_p", -1.0),
                           n=s.get("n", 1), best_of=s.get("best_of"))[0]
        gi.noise_fn = None
        if [g_["tokens"] for g_ in got] == [w["tokens"] for w in want]:
            same += 1
            for g_rec, w_rec in zip(got, want):
                assert all(abs(a - b) < 2e-2 for a, b in zip(g_rec["token_scores"],
                                                             w_rec["token_scores"])), s
    print("shared prefills (%s): %d / %d requests identical to their own generation"
          % (shared, same, len(specs)), flush=True)
    assert same >= len(specs) - 3
    assert cb.cache.lens.tolist() == [-1] * 12


def test_continuous_batcher_random_request_mix_equals_single_requests():
    """Forty requests with options drawn at random from everything the engine serves
    (temperature, top-p, decaying nucleus, the four penalty weights, logprobs, echo, replicas,
    minimum / maximum lengths, stop lists) over six slots that are reused many times: whatever
    a slot's previous occupant left behind, each request gets the tokens and scores of a
    generation of its own (lone prefills: to the last bit)."""
    from metaseq_amd.service import ContinuousBatcher
    cfg = tiny_cfg(layers=2, dim=128, heads=2, vocab=64, max_pos=48)
    sd = random_state_dict(cfg, seed=33, dtype=torch.float16)
    model = TransformerLanguageModel.build_model(cfg, sd, device=DEV)
    gi = GeneratorInterface(model, Dictionary(cfg.vocab_size, symbols={".": 13, "?": 29, "!": 41}))
    g = torch.Generator().manual_seed(77)

    def coin(p):
        return float(torch.rand(1, generator=g)) < p

    def pick(values):
        return values[int(torch.randint(0, len(values), (1,), generator=g))]
    specs = []
    for i in range(40):
        n = int(torch.randint(1, 10, (1,), generator=g))
        s = dict(prompt=torch.randint(4, 64, (n,), generator=g).tolist(),
                 max_tokens=int(torch.randint(2, 14, (1,), generator=g)))
        if coin(0.5):
            s.update(top_p=pick([0.3, 0.7, 0.95]), temperature=pick([0.7, 1.0, 1.3]))
            if coin(0.4):
                s.update(lambda_decay=pick([0.5, 0.8]), omega_bound=pick([0.1, 0.3]))
        elif coin(0.3):
            s.update(temperature=pick([0.0, 0.6]))
        if coin(0.3):
            s.update(alpha_presence=pick([0.0, 0.6]), alpha_frequency=pick([0.2, 0.5]))
        if coin(0.2):
            s.update(alpha_presence_src=0.5, alpha_frequency_src=pick([0.0, 0.3]),
                     alpha_src_penalty_end_idx=pick([-1, 2]))
        if coin(0.3):
            s.update(logprobs=pick([1, 4]), echo=coin(0.5))
        if coin(0.2):
            s.update(n=2, best_of=pick([2, 3]))
        if coin(0.3):
            s.update(min_tokens=min(3, s["max_tokens"]))
        if coin(0.15):
            s.update(stop=[pick([20, 33])])
        specs.append(s)
    cb = ContinuousBatcher(gi, slots=6, capacity=30,
                           noise_fn=lambda req, j, pos, V: _noise_for(req.prompt, j, pos, V))
    replies = [cb.submit(s["prompt"], **{k: v for k, v in s.items() if k != "prompt"})
               for s in specs]
    n = 0
    while cb.step():
        n += 1
        assert n < 1000
    for s, r in zip(specs, replies):
        _, got = r.get_nowait()
        assert not isinstance(got, Exception), (s, got)
        prompt = s["prompt"]
        gi.noise_fn = lambda step, BB, V: torch.stack(
            [_noise_for(prompt, j, step, V) for j in range(BB)])
        kw = {k: v for k, v in s.items() if k not in ("prompt", "max_tokens", "min_tokens")}
        want = gi.generate([prompt], max_tokens=[s["max_tokens"]],
                           min_tokens=[s.get("min_tokens", 0)], **kw)[0]
        gi.noise_fn = None
        assert len(got) == len(want)
        for g_rec, w_rec in zip(got, want):
            assert g_rec["tokens"] == w_rec["tokens"], (s, g_rec["tokens"], w_rec["tokens"])
            assert g_rec["token_scores"] == w_rec["token_scores"], s
            if s.get("logprobs"):
                for g_top, w_top in zip(g_rec["top_logprobs"], w_rec["top_logprobs"]):
                    assert (g_top is None) == (w_top is None)
                    if w_top is not None:
                        assert sorted(g_top.values()) == sorted(w_top.values()), s
    assert cb.cache.lens.tolist() == [-1] * 6
