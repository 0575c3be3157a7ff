"""Host logic of the serving loops: the run-to-completion service against a recording fake
generator (cost model, per-signature backlogs, budget and overflow rules, result routing, error
propagation) and the continuous batcher against a scripted fake decoder (slot bookkeeping,
per-row minimum / maximum / stop rules, records)."""
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


def _choose(last, length, mode, stop):
    t = _rule(last, length)
    if mode & 2:
        return EOS
    if mode & 1 and (t == EOS or t in stop):
        return ALT
    return t


class FakeSlotDecoder:
    """Stands in for TransformerDecoder's slot interface on the CPU."""

    class Cache:
        def __init__(self, slots):
            self.lens = [-1] * slots

    def __init__(self):
        self.prefills, self.steps = [], []

    def max_positions(self):
        return 64

    def new_slot_cache(self, slots, capacity, device=None):
        self.capacity = capacity
        return self.Cache(slots)

    def admit_slot(self, cache, slot, tokens, *, banned, stop, eos, mode, tok_out, score_out):
        assert cache.lens[slot] == -1 and banned == [PAD] and eos == EOS
        ids = tokens.tolist()
        self.prefills.append((slot, ids))
        cache.lens[slot] = len(ids)
        tok_out[0] = _choose(ids[-1], len(ids), mode, stop)
        score_out[0] = -0.5
        return [0.0] + [-1.0] * (len(ids) - 1)

    def decode_slots(self, cache, last_tokens, *, temperature, banned, stop, eos, row_mode,
                     tok_out, score_out):
        active = [i for i, n in enumerate(cache.lens) if n >= 0]
        self.steps.append(active)
        for i in active:
            assert cache.lens[i] < self.capacity, "a row outgrew its slot"
            cache.lens[i] += 1
            tok_out[i] = _choose(int(last_tokens[i]), cache.lens[i], int(row_mode[i]), stop)
            score_out[i] = -0.25

    def release_slot(self, cache, slot):
        cache.lens[slot] = -1


def _expected(prompt, min_tokens=0, max_tokens=0, stop=(), capacity=64):
    """What one request generates on its own: the loop written out."""
    ids = [EOS] + list(prompt)
    room = capacity - len(ids)
    max_new = max(1, min(max_tokens or room, room))
    out = []
    while True:
        mode = (1 if len(out) < min_tokens else 0) | (2 if len(out) >= max_new - 1 else 0)
        t = _choose(ids[-1], len(ids), mode, stop)
        out.append(t)
        if t == EOS or t in stop or len(out) >= max_new:
            return out
        ids.append(t)


def _batcher(slots=3, capacity=64):
    class Model:
        pass
    model = Model()
    model.decoder = FakeSlotDecoder()
    model.max_positions = model.decoder.max_positions
    gi = GeneratorInterface(model, Dictionary(V), device="cpu")
    return ContinuousBatcher(gi, slots=slots, capacity=capacity), model.decoder


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
    for bad in (dict(temperature=0.7, top_p=0.9), dict(n=2), dict(logprobs=3),
                dict(alpha_presence=0.5)):
        res = cb.submit([5], **bad).get_nowait()[1]
        assert isinstance(res, ValueError), bad
    assert isinstance(cb.submit([5] * 70).get_nowait()[1], ValueError)    # longer than a slot
    assert cb.step() == 0


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
