"""Host logic of the serving loops: the run-to-completion service against a recording fake
generator (cost model, per-signature backlogs, budget and overflow rules, result routing, error
propagation) and the continuous batcher against a scripted fake decoder (slot bookkeeping,
per-row minimum / maximum / stop rules, records)."""
import random
import threading

import pytest
import torch

from metaseq_amd import Dictionary, GeneratorInterface
from metaseq_amd.service import (BatchingService, ContinuousBatcher, Rectangle, Request, SlotBatch,
                                 prompt_cost)


class FakeGenerator:
    def __init__(self, fail=None):
        self.calls, self.fail = [], fail

    def generate(self, **kw):
        self.calls.append(kw)
        if self.fail is not None:
            raise self.fail
        return [[{"text": "len%d" % len(x), "n": kw.get("n", 1)}] for x in kw["inputs"]]


def test_cost_model_and_ordering():
    # workers.py:57-59: n + ceil((n / 10) ** 2)
    assert [prompt_cost(n) for n in (0, 1, 10, 25, 100)] == [0, 2, 11, 32, 200]
    a = Request(1, [1] * 4, {}), Request(0, [1] * 4, {}), Request(9, [1] * 2, {})
    order = sorted(a, key=lambda r: r.rank)
    assert [r.uid for r in order] == [9, 0, 1] and a[0].cost == 5


def test_rectangle_owns_the_budget_and_overflow_arithmetic():
    box = Rectangle(token_budget=100, max_seq_len=64)
    first = Request(0, [1] * 30, {"max_tokens": 200})
    assert box.fits(first)            # a lone request is never refused by the planner
    box.add(first)
    assert not box.fits(Request(1, [1] * 2, {"max_tokens": 1}))     # 30 + 200 > 64
    box = Rectangle(token_budget=100, max_seq_len=64)
    box.add(Request(0, [1] * 20, {"max_tokens": 4}))                # cost 24
    assert box.fits(Request(1, [1] * 20, {"max_tokens": 4}))        # 24 * 2 <= 100
    box.add(Request(1, [1] * 20, {"max_tokens": 4}))
    box.add(Request(2, [1] * 20, {"max_tokens": 4}))
    box.add(Request(3, [1] * 20, {"max_tokens": 4}))                # 24 * 4 = 96
    assert not box.fits(Request(4, [1] * 2, {"max_tokens": 4}))     # 24 * 5 > 100
    args = box.call_arguments(seed=7)
    assert args["seed"] == 7 and args["max_tokens"] == [4] * 4 and len(args["inputs"]) == 4


def test_batches_group_by_signature_and_respect_the_token_budget():
    gen = FakeGenerator()
    svc = BatchingService(gen, max_tokens=100, timeout_ms=5, seed=1)
    rets = [svc.submit([1] * n, max_tokens=4, temperature=1.0, top_p=0.9)
            for n in (30, 4, 10, 20)]
    other = svc.submit([1] * 5, max_tokens=4, temperature=0.7, top_p=0.9)   # another signature
    sizes = []
    while True:
        n = svc.step()
        if n == 0:
            break
        sizes.append(n)
    # fullest queue first, cheapest first: costs 6, 11, 24 fit (24 * 3 = 72 <= 100); adding 39
    # would cost 39 * 4 = 156 > 100 -> next batch; then the other signature
    assert sizes == [3, 1, 1]
    assert [len(x) for x in gen.calls[0]["inputs"]] == [4, 10, 20]
    assert [len(x) for x in gen.calls[1]["inputs"]] == [30]
    assert gen.calls[2]["temperature"] == 0.7 and gen.calls[0]["temperature"] == 1.0
    assert gen.calls[0]["max_tokens"] == [4, 4, 4] and gen.calls[0]["min_tokens"] == [0, 0, 0]
    assert 1 <= gen.calls[0]["seed"] <= 20000
    # every caller gets its own result, keyed by its uid
    for n, r in zip((30, 4, 10, 20), rets):
        uid, res = r.get_nowait()
        assert res[0]["text"] == "len%d" % n
    assert other.get_nowait()[1][0]["text"] == "len5"


def test_sequence_length_overflow_splits_a_batch():
    gen = FakeGenerator()
    svc = BatchingService(gen, max_tokens=10 ** 9, max_seq_len=64, timeout_ms=5)
    svc.submit([1] * 10, max_tokens=50)     # 10 + 50 fits
    svc.submit([1] * 20, max_tokens=10)     # max prompt 20 + max gen 50 = 70 > 64
    assert svc.step() == 1 and svc.step() == 1 and svc.step() == 0
    assert [len(c["inputs"]) for c in gen.calls] == [1, 1]


def test_exceptions_are_reported_and_device_faults_propagate():
    svc = BatchingService(FakeGenerator(fail=ValueError("bad request")), timeout_ms=5)
    r = svc.submit([1, 2, 3])
    assert svc.step() == 1
    uid, res = r.get_nowait()
    assert isinstance(res, ValueError)
    svc = BatchingService(FakeGenerator(fail=RuntimeError("device lost")), timeout_ms=5)
    svc.submit([1, 2, 3])
    with pytest.raises(RuntimeError):
        svc.step()


def test_serving_thread_answers_blocking_callers():
    gen = FakeGenerator()
    svc = BatchingService(gen, timeout_ms=10)
    t = threading.Thread(target=svc.serve_forever, daemon=True)
    t.start()
    out = {}

    def call(n):
        out[n] = svc.generate([7] * n, max_tokens=2)
    callers = [threading.Thread(target=call, args=(n,)) for n in (3, 5, 8)]
    for c in callers:
        c.start()
    for c in callers:
        c.join(timeout=10)
    svc.stop()
    t.join(timeout=10)
    assert not t.is_alive()
    assert {n: out[n][0]["text"] for n in out} == {3: "len3", 5: "len5", 8: "len8"}
    assert sum(len(c["inputs"]) for c in gen.calls) == 3


# ---- continuous batching against a scripted decoder ----------------------------------------------
V, EOS, PAD, ALT = 50, 2, 1, 7


def _rule(last, length):
    """The scripted model: the next token is a fixed function of the last token and of how
    many positions the row holds; now and then it is the end-of-sequence token."""
    t = (last * 11 + length * 5) % V
    return EOS if t % 9 == 0 else max(t, 4)


def _choose(last, length, mode, stop, temperature=1.0, topp=0.0, noise=None, penalty=0):
    """A row of the scripted model.  Rows that are not plainly greedy shift the rule's token by
    a function of their temperature, of their nucleus and, when they sample, of the largest
    noise entry, and by ``penalty``: what matters to these tests is that every parameter
    reaches the row it belongs to."""
    t = _rule(last, length)
    if temperature != 1.0 or topp > 0 or penalty:
        shift = int(round(temperature * 10)) + penalty
        if topp > 0:
            shift += int(noise.argmax()) + int(round(topp * 100))
        t = max((t + shift) % V, 4)
    if mode & 2:
        return EOS
    if mode & 1 and (t == EOS or t in stop):
        return ALT
    return t


def _penalty(alphas, counts, counts_src, last):
    """The scripted model's use of the penalty state of a row: its four weights, how many
    tokens it has generated, and how often its last token occurs in the prompt."""
    if max(alphas) <= 0:
        return 0
    return (int(round(sum(a * w for a, w in zip(alphas, (10, 20, 30, 40)))))
            + int(counts.sum()) + 3 * int(counts_src[last]))


def _lprob_row(tok):
    """The scripted model's log-probabilities of a step that chose ``tok``: no two alike."""
    return -((torch.arange(V) * 7 + tok) % V).float()


class FakeSlotDecoder:
    """Stands in for TransformerDecoder's slot interface on the CPU."""

    class Cache:
        def __init__(self, slots):
            self.lens = [-1] * slots

    def __init__(self):
        self.prefills, self.steps, self.shared = [], [], []

    def admit_slots(self, cache, requests):
        self.shared.append(len(requests))
        out = []
        for r in requests:
            kw = {k: v for k, v in r.items() if k not in ("slot", "tokens")}
            out.append(self.admit_slot(cache, r["slot"], r["tokens"], **kw))
        return out

    def max_positions(self):
        return 64

    def new_slot_cache(self, slots, capacity, device=None):
        self.capacity = capacity
        return self.Cache(slots)

    def admit_slot(self, cache, slot, tokens, *, banned, stop, eos, mode, tok_out, score_out,
                   temperature=1.0, topp=0.0, noise=None, replicas=(), penalties=None,
                   lprobs_out=None, prompt_topk=0, detail=None):
        assert banned == [PAD] and eos == EOS
        ids = tokens.tolist()
        self.prefills.append((slot, ids))
        for r, s in enumerate([slot] + list(replicas)):
            assert cache.lens[s] == -1
            cache.lens[s] = len(ids)
            pen = 0
            if penalties is not None:
                assert int(penalties["counts"][r].sum()) == 0
                pen = _penalty(penalties["alphas"], penalties["counts"][r],
                               penalties["counts_src"][r], ids[-1])
            t = _choose(ids[-1], len(ids), mode, stop, temperature, topp,
                        None if noise is None else noise[r], pen)
            tok_out[r] = t
            score_out[r] = -0.5 - 0.01 * r
            if penalties is not None:
                penalties["counts"][r, t] += 1
            if lprobs_out is not None:
                lprobs_out[r] = _lprob_row(t)
        if prompt_topk:
            rows = torch.stack([_lprob_row(t) for t in ids[1:]])
            values, top = rows.topk(prompt_topk, dim=-1)
            detail["prompt_top"] = (values, top)
        return [0.0] + [-1.0] * (len(ids) - 1)

    def decode_slots(self, cache, last_tokens, *, temperature, banned, stop, eos, row_mode,
                     tok_out, score_out, logits_out=None, sampled=None):
        active = [i for i, n in enumerate(cache.lens) if n >= 0]
        self.steps.append(active)
        for i in active:
            assert cache.lens[i] < self.capacity, "a row outgrew its slot"
            cache.lens[i] += 1
            tok_out[i] = _choose(int(last_tokens[i]), cache.lens[i], int(row_mode[i]), stop)
            score_out[i] = -0.25
        if sampled is not None:
            assert logits_out is not None
            for i in active:
                m = int(sampled["row_mode"][i])
                if m & 4:
                    continue
                topp = float(sampled["topp"][i])
                pen = 0
                if sampled.get("penalty_rows") is not None:
                    pen = _penalty([round(float(a), 4) for a in sampled["penalty_rows"][i]],
                                   sampled["counts"][i], sampled["counts_src"][i],
                                   int(last_tokens[i]))
                t = _choose(int(last_tokens[i]), cache.lens[i], m, stop,
                            round(float(sampled["temperature"][i]), 4), round(topp, 4),
                            sampled["noise"][i] if topp > 0 else None, pen)
                tok_out[i] = t
                score_out[i] = -0.125 * (i + 1)
                if sampled.get("penalty_rows") is not None:
                    sampled["counts"][i, t] += 1
                if sampled.get("lprobs_out") is not None:
                    sampled["lprobs_out"][i] = _lprob_row(t)

    def release_slot(self, cache, slot):
        cache.lens[slot] = -1


def _expected(prompt, min_tokens=0, max_tokens=0, stop=(), capacity=64, temperature=1.0,
              topp=0.0, noise=None, alphas=(0.0, 0.0, 0.0, 0.0), src_end=-1, decay=-1.0,
              omega=0.3, full_stop=(), top=None):
    """What one request generates on its own: the loop written out.  ``noise(position)`` gives
    the row's Exp(1) numbers for the draw of the token at that position; ``top`` (a list)
    receives the scripted log-probability row of every step."""
    ids = [EOS] + list(prompt)
    room = capacity - len(ids)
    max_new = max(1, min(max_tokens or room, room))
    counts = torch.zeros(V, dtype=torch.long)
    counts_src = torch.zeros(V, dtype=torch.long)
    for t in (ids if src_end <= 0 else ids[:src_end]):
        counts_src[t] += 1
    since, out = 0, []
    while True:
        mode = (1 if len(out) < min_tokens else 0) | (2 if len(out) >= max_new - 1 else 0)
        p = topp
        if decay > 0 and topp > 0:   # fp32, as the generation loop computes it
            p = float(torch.clamp(torch.tensor(topp) * torch.tensor(decay) ** max(since - 1, 0),
                                  min=omega))
        t = _choose(ids[-1], len(ids), mode, stop, temperature, round(p, 4),
                    noise(len(ids)) if (noise and topp > 0) else None,
                    _penalty(alphas, counts, counts_src, ids[-1]))
        counts[t] += 1
        since = 0 if t in full_stop else since + 1
        if top is not None:
            top.append(_lprob_row(t))
        out.append(t)
        if t == EOS or t in stop or len(out) >= max_new:
            return out
        ids.append(t)


def _batcher(slots=3, capacity=64, symbols=None, **kw):
    class Model:
        pass
    model = Model()
    model.decoder = FakeSlotDecoder()
    model.max_positions = model.decoder.max_positions
    gi = GeneratorInterface(model, Dictionary(V, symbols=symbols), device="cpu")
    return ContinuousBatcher(gi, slots=slots, capacity=capacity, **kw), model.decoder


def _drain(cb, limit=500):
    n = 0
    while cb.step():
        n += 1
        assert n < limit
    return n


def test_slot_batch_caps_new_tokens_by_what_the_slot_holds():
    sb = SlotBatch(slots=2, capacity=16)
    assert sb.room_for(Request(0, [5] * 5, {"max_tokens": 4})) == 4
    assert sb.room_for(Request(0, [5] * 5, {"max_tokens": 100})) == 10    # 16 - (5 + 1)
    assert sb.room_for(Request(0, [5] * 5, {})) == 10
    assert sb.room_for(Request(0, [5] * 15, {})) == 0                     # the prompt fills it
    assert sb.free_slot() == 0


def test_continuous_batcher_gives_every_request_its_own_single_request_result():
    """More requests than slots, different prompt lengths, minimum and maximum lengths: rows
    join and leave while the others keep decoding, and every answer equals what the request
    generates alone."""
    cb, dec = _batcher(slots=3)
    specs = [dict(prompt=[5, 9, 4], max_tokens=12), dict(prompt=[8], max_tokens=3),
             dict(prompt=[6] * 10, min_tokens=6, max_tokens=20), dict(prompt=[17, 4], max_tokens=1),
             dict(prompt=[21, 30, 12, 9], min_tokens=2, max_tokens=9),
             dict(prompt=[33], max_tokens=30), dict(prompt=[4, 4, 4, 4, 4, 4], max_tokens=7)]
    replies = [cb.submit(s["prompt"], **{k: v for k, v in s.items() if k != "prompt"})
               for s in specs]
    _drain(cb)
    for s, r in zip(specs, replies):
        _, res = r.get_nowait()
        want = _expected(**s)
        shown = [t for t in want if t != EOS]
        assert res[0]["tokens"] == [str(t) for t in shown], (s, res[0]["tokens"], want)
        assert res[0]["text"] == " ".join(str(t) for t in shown)
        assert len(res[0]["token_scores"]) == len(shown)
    # rows really overlapped: some step served several rows, and slots were reused
    assert max(len(a) for a in dec.steps) == 3 and len(dec.prefills) == len(specs)
    assert len({slot for slot, _ in dec.prefills}) == 3
    assert cb.rows_stepped == sum(len(a) for a in dec.steps)
    # cheapest prompts were admitted first
    assert [len(ids) - 1 for _, ids in dec.prefills[:3]] == [1, 1, 2]


def test_continuous_batcher_echo_stop_lists_and_refusals():
    cb, dec = _batcher(slots=2)
    # echo returns the prompt too, with a withheld score for the leading end-of-sequence token
    r = cb.submit([5, 9, 4], max_tokens=4, echo=True)
    _drain(cb)
    res = r.get_nowait()[1][0]
    want = [t for t in _expected([5, 9, 4], max_tokens=4) if t != EOS]
    assert res["tokens"] == ["2", "5", "9", "4"] + [str(t) for t in want]
    assert res["token_scores"][0] is None and res["token_scores"][1:4] == [-1.0, -1.0, -1.0]
    # a stop token ends its row and stays in the output; another stop list waits for the drain
    first = _expected([8, 8], max_tokens=30)
    stop = [first[2]]
    a = cb.submit([8, 8], max_tokens=30, stop=stop)
    b = cb.submit([8, 8, 8], max_tokens=5)
    _drain(cb)
    assert a.get_nowait()[1][0]["tokens"] == [str(t) for t in first[:3]]
    assert b.get_nowait()[1][0]["tokens"] == [
        str(t) for t in _expected([8, 8, 8], max_tokens=5) if t != EOS]
    assert all(len(act) == 1 for act in dec.steps[-8:])   # the two never shared a step
    # what the engine does not serve is answered with an error, not queued
    for bad in (dict(logprobs=V + 1), dict(lambda_decay=0.9, top_p=0.5), dict(n=3),
                dict(n=2, best_of=1), dict(temperature=-1)):   # no "." in this dictionary
        res = cb.submit([5], **bad).get_nowait()[1]
        assert isinstance(res, ValueError), bad
    assert isinstance(cb.submit([5] * 70).get_nowait()[1], ValueError)    # longer than a slot
    assert cb.step() == 0


def _noise(req, replica, position, vocab):
    """Exp(1)-like numbers that depend on nothing but the request's prompt, the replica and the
    position of the token being drawn."""
    g = torch.Generator().manual_seed(1000 * sum(req.prompt) + 100 * replica + position)
    return torch.empty(vocab).exponential_(generator=g)


def test_continuous_batcher_mixes_greedy_and_sampled_rows_each_under_its_own_parameters():
    """Sampled requests (their own temperature and top-p), greedy ones at another temperature
    and plainly greedy ones share the running batch; every row is chosen with its own
    parameters and noise, so each answer equals the request's own single-request loop."""
    cb, dec = _batcher(slots=4, noise_fn=_noise)
    specs = [dict(prompt=[5, 9, 4], max_tokens=12, temperature=0.7, top_p=0.9),
             dict(prompt=[8], max_tokens=9),
             dict(prompt=[6] * 7, min_tokens=4, max_tokens=15, temperature=1.3, top_p=0.5),
             dict(prompt=[17, 4], max_tokens=8, temperature=0.5),                  # greedy, scaled
             dict(prompt=[21, 30], max_tokens=10, temperature=0, top_p=0.9),      # plainly greedy
             dict(prompt=[33, 13], max_tokens=11, top_p=0.3)]
    replies = [cb.submit(s["prompt"], **{k: v for k, v in s.items() if k != "prompt"})
               for s in specs]
    _drain(cb)
    assert max(len(a) for a in dec.steps) == 4
    for s, r in zip(specs, replies):
        res = r.get_nowait()[1]
        assert not isinstance(res, Exception), res
        t, p = s.get("temperature", 1.0), s.get("top_p", -1.0)
        t, p = (1.0, 0.0) if t == 0 else (t, max(p, 0.0))
        req = Request(0, s["prompt"], {})
        want = _expected(s["prompt"], s.get("min_tokens", 0), s["max_tokens"], temperature=t,
                         topp=p, noise=lambda pos: _noise(req, 0, pos, V))
        assert res[0]["tokens"] == [str(x) for x in want if x != EOS], (s, res[0]["tokens"], want)


def test_continuous_batcher_replicas_share_one_prefill_and_come_back_best_first():
    cb, dec = _batcher(slots=4, noise_fn=_noise)
    a = cb.submit([5, 9, 4], max_tokens=6, temperature=0.9, top_p=0.8, n=2, best_of=3)
    b = cb.submit([8, 8], max_tokens=5)
    _drain(cb)
    assert len(dec.prefills) == 2                       # one prefill per request
    res = a.get_nowait()[1]
    assert len(res) == 2
    req = Request(0, [5, 9, 4], {})
    runs = []
    for j in range(3):
        toks = _expected([5, 9, 4], max_tokens=6, temperature=0.9, topp=0.8,
                         noise=lambda pos: _noise(req, j, pos, V))
        runs.append([str(x) for x in toks if x != EOS])
    got = [r["tokens"] for r in res]
    assert all(g in runs for g in got)
    sums = [sum(r["token_scores"]) for r in res]
    assert sums[0] >= sums[1]
    assert b.get_nowait()[1][0]["tokens"] == [
        str(t) for t in _expected([8, 8], max_tokens=5) if t != EOS]
    # three replicas wait until three slots are free at once
    cb, dec = _batcher(slots=3, noise_fn=_noise)
    first = cb.submit([9] * 4, max_tokens=20)
    second = cb.submit([7, 7, 7, 7, 7, 7, 7, 7], max_tokens=4, top_p=0.9, best_of=3)
    _drain(cb)
    assert len(second.get_nowait()[1]) == 1 and len(first.get_nowait()[1]) == 1
    assert all(len(a) <= 3 for a in dec.steps)


def test_continuous_batcher_serves_a_request_that_has_waited_before_cheaper_ones():
    """Cheapest first is the rule, but a request that has waited ``patience`` steps goes first,
    and a request whose stop list differs from the running batch's blocks later arrivals until
    the batch has drained: neither can starve."""
    cb, dec = _batcher(slots=1, patience=3)
    long_one = cb.submit([9] * 12, max_tokens=2)
    for _ in range(12):
        cb.submit([8], max_tokens=2)                    # cheaper, keeps arriving first in rank
    order = []
    for _ in range(60):
        before = len(dec.prefills)
        if not cb.step():
            break
        order += [len(ids) - 1 for _, ids in dec.prefills[before:]]
    assert long_one.get_nowait()[1][0] is not None
    assert order.index(12) <= 3                         # not after all twelve cheap ones


def test_continuous_batcher_serving_thread():
    cb, _ = _batcher(slots=2)
    t = threading.Thread(target=cb.serve_forever, daemon=True)
    t.start()
    out = {}

    def call(n):
        out[n] = cb.generate([9] * n, max_tokens=6)
    callers = [threading.Thread(target=call, args=(n,)) for n in (1, 2, 3, 4, 5)]
    for c in callers:
        c.start()
    for c in callers:
        c.join(timeout=20)
    cb.stop()
    t.join(timeout=10)
    assert not t.is_alive() and sorted(out) == [1, 2, 3, 4, 5]
    for n in out:
        want = [str(x) for x in _expected([9] * n, max_tokens=6) if x != EOS]
        assert out[n][0]["tokens"] == want


FULL_STOPS = {".": 13, "?": 29, "!": 41}


def test_continuous_batcher_penalties_decaying_nucleus_and_alternatives_per_row():
    """Requests with repetition penalties (own weights, prompt counts cut at
    alpha_src_penalty_end_idx), with a decaying nucleus, with ``logprobs`` and with none of
    these share the running batch; slots are reused by requests of another kind.  Every answer
    equals the request's own loop, and the alternatives reported per position are those of the
    step that chose the token there."""
    cb, dec = _batcher(slots=3, symbols=FULL_STOPS, noise_fn=_noise)
    specs = [
        dict(prompt=[5, 9, 5, 5], max_tokens=10, alpha_presence=0.5, alpha_frequency=0.2),
        dict(prompt=[8, 8, 8], max_tokens=12, temperature=0.8, top_p=0.9, lambda_decay=0.7,
             omega_bound=0.4),
        dict(prompt=[6] * 5, max_tokens=9, logprobs=3),
        dict(prompt=[17, 4, 17, 17], max_tokens=8, alpha_presence_src=0.3,
             alpha_frequency_src=0.1, alpha_src_penalty_end_idx=3, top_p=0.6, logprobs=2,
             echo=True),
        dict(prompt=[21, 30], max_tokens=10),
        dict(prompt=[33, 13, 2 + 9], max_tokens=14, top_p=0.8, lambda_decay=0.5, min_tokens=3,
             alpha_frequency=0.4),
    ]
    replies = [cb.submit(s["prompt"], **{k: v for k, v in s.items() if k != "prompt"})
               for s in specs]
    _drain(cb)
    assert max(len(a) for a in dec.steps) == 3 and len({slot for slot, _ in dec.prefills}) == 3
    for s, r in zip(specs, replies):
        res = r.get_nowait()[1]
        assert not isinstance(res, Exception), (s, res)
        req = Request(0, s["prompt"], {})
        top = []
        want = _expected(
            s["prompt"], s.get("min_tokens", 0), s["max_tokens"],
            temperature=s.get("temperature", 1.0), topp=max(s.get("top_p", 0.0), 0.0),
            noise=lambda pos: _noise(req, 0, pos, V),
            alphas=tuple(s.get(k, 0.0) for k in ("alpha_presence", "alpha_frequency",
                                                 "alpha_presence_src", "alpha_frequency_src")),
            src_end=s.get("alpha_src_penalty_end_idx", -1), decay=s.get("lambda_decay", -1.0),
            omega=s.get("omega_bound", 0.3), full_stop=tuple(FULL_STOPS.values()), top=top)
        shown = [t for t in want if t != EOS]
        lead = [str(t) for t in [EOS] + s["prompt"]] if s.get("echo") else []
        assert res[0]["tokens"] == lead + [str(t) for t in shown], (s, res[0]["tokens"], want)
        k = s.get("logprobs", 0)
        if not k:
            assert res[0]["top_logprobs"] is None
            continue
        rows = top[:len(shown)]
        if s.get("echo"):   # the prompt's positions: nothing for the leading token
            assert res[0]["top_logprobs"][0] is None
            rows = [_lprob_row(t) for t in s["prompt"]] + rows
        got = res[0]["top_logprobs"][1:] if s.get("echo") else res[0]["top_logprobs"]
        assert len(got) == len(rows)
        for g, row in zip(got, rows):
            values, ids = row.topk(k)
            assert g == {str(i): v for i, v in zip(ids.tolist(), values.tolist())}


def test_continuous_batcher_shares_prefills_and_waits_for_company():
    """prefill_batch > 1: the requests admitted in one step share one prefill; with
    prefill_wait a lone admissible request is held back, while rows are decoding, until others
    can join it or the wait is over.  Every answer still equals the request's own loop."""
    cb, dec = _batcher(slots=4, noise_fn=_noise, prefill_batch=3, prefill_wait=2)
    specs = [dict(prompt=[5, 9, 4], max_tokens=12), dict(prompt=[8], max_tokens=3),
             dict(prompt=[6] * 10, min_tokens=6, max_tokens=20, temperature=0.7, top_p=0.9),
             dict(prompt=[17, 4], max_tokens=2), dict(prompt=[21, 30, 12, 9], max_tokens=9),
             dict(prompt=[33], max_tokens=30, top_p=0.5), dict(prompt=[4, 4, 4, 4], max_tokens=7),
             dict(prompt=[40, 41], max_tokens=5), dict(prompt=[44], max_tokens=11)]
    replies = [cb.submit(s["prompt"], **{k: v for k, v in s.items() if k != "prompt"})
               for s in specs]
    _drain(cb)
    for s, r in zip(specs, replies):
        res = r.get_nowait()[1]
        assert not isinstance(res, Exception), res
        req = Request(0, s["prompt"], {})
        want = _expected(s["prompt"], s.get("min_tokens", 0), s["max_tokens"],
                         temperature=s.get("temperature", 1.0), topp=max(s.get("top_p", 0.0), 0.0),
                         noise=lambda pos: _noise(req, 0, pos, V))
        assert res[0]["tokens"] == [str(t) for t in want if t != EOS], (s, res[0]["tokens"])
    assert len(dec.prefills) == len(specs)
    assert dec.shared[0] == 3                       # the first three at once
    assert sum(dec.shared) + (len(dec.prefills) - sum(dec.shared)) == len(specs)
    assert len(dec.shared) >= 2 and max(dec.shared) <= 3
    # a request arriving while rows decode waits at most prefill_wait steps for company
    cb, dec = _batcher(slots=4, prefill_batch=3, prefill_wait=2)
    first = cb.submit([6] * 5, max_tokens=30, min_tokens=30)
    cb.step()
    late = cb.submit([7, 7], max_tokens=4)
    cb.step(), cb.step()
    assert len(dec.prefills) == 1                   # held back twice
    cb.step()
    assert len(dec.prefills) == 2                   # then admitted alone
    _drain(cb)
    assert not isinstance(first.get_nowait()[1], Exception)
    assert late.get_nowait()[1][0]["tokens"] == [
        str(t) for t in _expected([7, 7], max_tokens=4) if t != EOS]


def test_shared_prefills_group_prompts_of_similar_length():
    """A shared prefill pads every prompt to its longest: groups are closed at prefill_batch
    members or when padding would exceed half of the real rows."""
    class Knobs:
        prefill_batch = 4
    groups = ContinuousBatcher._prefill_groups(
        Knobs(), [dict(ids=[0] * n) for n in (5, 6, 7, 100, 8, 120, 110, 9, 300)])
    assert [[len(p["ids"]) for p in g] for g in groups] == [[5, 6, 7, 8], [9], [100, 110, 120],
                                                            [300]]
    Knobs.prefill_batch = 1
    groups = ContinuousBatcher._prefill_groups(Knobs(), [dict(ids=[0] * n) for n in (3, 3, 3)])
    assert [len(g) for g in groups] == [1, 1, 1]


@pytest.mark.parametrize("seed,slots,prefill", [(1, 2, (1, 0)), (2, 3, (3, 2)), (3, 5, (4, 1)),
                                                (4, 1, (1, 0)), (5, 7, (2, 5))])
def test_continuous_batcher_random_traffic_against_the_scripted_model(seed, slots, prefill):
    """150 requests with random prompts, length limits, temperatures, nuclei (fixed and
    decaying), penalties, replicas and two stop lists, arriving in bursts while the engine
    runs, over few slots: every answer equals the request's own loop.  The engine queues each
    decode step before it reads the previous one, so rows that have just ended are stepped once
    more, slots change hands between two reads, and requests with another stop list wait for
    the batch to drain - none of which may show in a result."""
    rng = random.Random(seed)
    cb, dec = _batcher(slots=slots, symbols=FULL_STOPS, noise_fn=_noise,
                       prefill_batch=prefill[0], prefill_wait=prefill[1], patience=20)
    specs, replies = [], []
    pending = 150
    steps = 0
    while True:
        busy = cb.step()
        if not (pending or busy or any(r.empty() for r in replies)):
            break
        steps += 1
        assert steps < 20000
        for _ in range(min(pending, rng.choice([0, 0, 0, 1, 2, 5]))):
            pending -= 1
            s = dict(prompt=[rng.randint(4, V - 1) for _ in range(rng.randint(1, 9))],
                     max_tokens=rng.randint(1, 14))
            if rng.random() < 0.5:
                s.update(temperature=rng.choice([0.7, 1.3]), top_p=rng.choice([0.4, 0.9]))
                if rng.random() < 0.4:
                    s.update(lambda_decay=rng.choice([0.5, 0.8]), omega_bound=0.2)
            elif rng.random() < 0.3:
                s.update(temperature=0.5)
            if rng.random() < 0.3:
                s.update(alpha_presence=0.5, alpha_frequency=rng.choice([0.0, 0.3]))
            if rng.random() < 0.2:
                s.update(alpha_frequency_src=0.2, alpha_src_penalty_end_idx=rng.choice([-1, 2]))
            if rng.random() < 0.3:
                s.update(min_tokens=min(rng.randint(1, 4), s["max_tokens"]))
            if rng.random() < 0.15:
                s.update(stop=[17, 23])
            if rng.random() < 0.15 and slots >= 2:
                s.update(n=1, best_of=2)
            specs.append(s)
            replies.append(cb.submit(s["prompt"],
                                     **{k: v for k, v in s.items() if k != "prompt"}))
    for s, r in zip(specs, replies):
        res = r.get_nowait()[1]
        assert not isinstance(res, Exception), (s, res)
        req = Request(0, s["prompt"], {})
        runs = []
        for j in range(s.get("best_of", 1)):
            want = _expected(
                s["prompt"], s.get("min_tokens", 0), s["max_tokens"], stop=s.get("stop", ()),
                temperature=s.get("temperature", 1.0), topp=max(s.get("top_p", 0.0), 0.0),
                noise=lambda pos, j=j: _noise(req, j, pos, V),
                alphas=(s.get("alpha_presence", 0.0), s.get("alpha_frequency", 0.0), 0.0,
                        s.get("alpha_frequency_src", 0.0)),
                src_end=s.get("alpha_src_penalty_end_idx", -1), decay=s.get("lambda_decay", -1.0),
                omega=s.get("omega_bound", 0.3), full_stop=tuple(FULL_STOPS.values()))
            runs.append([str(t) for t in want if t != EOS])
        assert res[0]["tokens"] in runs, (s, res[0]["tokens"], runs)
    assert all(n < 0 for n in cb.cache.lens)
