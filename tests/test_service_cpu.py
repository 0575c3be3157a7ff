"""Host logic of the dynamic-batching service against a recording fake generator: cost model,
per-signature queues, budget and overflow rules, result routing, error propagation."""
import queue
import threading

import pytest

from metaseq_amd.service import BatchingService, WorkItem, prompt_cost


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
    a = WorkItem(5, 1, None, {}), WorkItem(5, 0, None, {}), WorkItem(3, 9, None, {})
    assert sorted(a)[0].uid == 9 and sorted(a)[1].uid == 0


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
