"""Dynamic batching in front of ``GeneratorInterface``: the work queue, cost model and batching
loop of the reference's hosted service (metaseq/service/queue.py, metaseq/service/workers.py,
metaseq/cli/interactive_hosted.py:66-175), without its web layer.

Requests are queued per generation-argument signature (requests that sample differently cannot
share a batch), served smallest-cost first from the fullest queue, and grouped until the padded
batch would exceed ``max_tokens`` or ``max_prompt + max_gen`` would exceed the model's sequence
length; an unfilled batch runs after ``timeout`` milliseconds.  One thread drives the GPU
(interactive_hosted.py:205); callers block on their own return queue.
"""
import math
import queue
import random
import threading
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

# arguments that must agree within a batch (metaseq/service/workers.py:13-23)
QUEUE_KEYS = ["temperature", "top_p", "n", "lambda_decay", "omega_bound", "alpha_presence",
              "alpha_frequency", "alpha_presence_src", "alpha_frequency_src"]
# arguments copied from the batch's requests into the generate() call
# (interactive_hosted.py:125-142)
SHARED_ARGS = ["temperature", "top_p", "n", "best_of", "echo", "logprobs", "stop", "omega_bound",
               "lambda_decay", "alpha_presence", "alpha_frequency", "alpha_presence_src",
               "alpha_frequency_src", "alpha_src_penalty_end_idx"]
MAX_SEQ_LEN = 2048        # metaseq/service/constants.py:8
MAX_BATCH_TOKENS = 3072   # metaseq/service/constants.py:10


def prompt_cost(n_tokens: int) -> int:
    """Linear layers plus attention (metaseq/service/workers.py:57-59)."""
    return n_tokens + int(math.ceil((n_tokens / 10) ** 2))


@dataclass(order=False)
class WorkItem:
    """Sortable queue entry: lower cost is served first, ties by uid
    (metaseq/service/workers.py:26-50)."""
    cost: int
    uid: int
    return_queue: "queue.Queue"
    data: Any
    prompt_len: int = 0
    gen_len: int = 0

    def __lt__(self, other):
        return (self.cost, self.uid) < (other.cost, other.uid)

    def __eq__(self, other):
        return (self.cost, self.uid) == (other.cost, other.uid)

    def queue_key(self) -> str:
        d = {k: self.data.get(k) for k in QUEUE_KEYS}
        return ":".join("%s:%s" % (k, d[k]) for k in sorted(d))


class KeyedQueues:
    """One priority queue per signature; the batching loop drains the fullest one
    (metaseq/service/queue.py:11-49)."""

    def __init__(self):
        self.queues: Dict[str, "queue.PriorityQueue"] = {}
        self._lock = threading.Lock()

    def put(self, item: WorkItem):
        with self._lock:
            q = self.queues.setdefault(item.queue_key(), queue.PriorityQueue())
        q.put(item)

    def get_largest_queue(self) -> Optional["queue.PriorityQueue"]:
        with self._lock:
            if not self.queues:
                return None
            key = max(self.queues, key=lambda k: self.queues[k].qsize())
            return self.queues[key]


class BatchingService:
    """``submit`` from any thread; ``serve_forever`` (or ``step``) on the one GPU thread."""

    def __init__(self, generator, max_tokens: int = MAX_BATCH_TOKENS,
                 max_seq_len: int = MAX_SEQ_LEN, timeout_ms: float = 100.0, seed: int = None):
        self.generator = generator
        self.max_tokens = max_tokens
        self.max_seq_len = max_seq_len
        self.timeout = timeout_ms / 1000.0
        self.queues = KeyedQueues()
        self._uid = 0
        self._uid_lock = threading.Lock()
        self._rng = random.Random(seed)
        self._stop = threading.Event()

    # -- producer side ----------------------------------------------------------------
    def submit(self, encoded_prompt: List[int], **generation_args) -> "queue.Queue":
        """Queues one prompt; the returned queue receives ``(uid, result_or_exception)``."""
        with self._uid_lock:
            uid = self._uid
            self._uid += 1
        ro = {"input": list(encoded_prompt), **generation_args}
        n = len(encoded_prompt)
        ret: "queue.Queue" = queue.Queue()
        self.queues.put(WorkItem(prompt_cost(n), uid, ret, ro, prompt_len=n,
                                 gen_len=int(ro.get("max_tokens", 0) or 0)))
        return ret

    def generate(self, encoded_prompt: List[int], **generation_args):
        """Blocking convenience call (metaseq/service/workers.py:52-62)."""
        _, result = self.submit(encoded_prompt, **generation_args).get()
        if isinstance(result, Exception):
            raise result
        return result

    # -- consumer side ----------------------------------------------------------------
    def collect_batch(self) -> List[WorkItem]:
        """Pulls like-sized items from the fullest queue until the padded batch is over budget
        (``longest cost x batch size > max_tokens``), would overflow the sequence length, or
        the queue stays empty for ``timeout`` (interactive_hosted.py:93-118)."""
        batch: List[WorkItem] = []
        target = self.queues.get_largest_queue()
        if target is None:
            return batch
        while True:
            try:
                item = target.get(timeout=self.timeout)
            except queue.Empty:
                return batch
            longest = max([item] + batch).cost
            batch_cost = longest * (len(batch) + 1)
            max_prompt_len = max(x.prompt_len for x in [item] + batch)
            max_gen_len = max(x.gen_len for x in [item] + batch)
            overflow = (max_prompt_len + max_gen_len) > self.max_seq_len
            if batch and (batch_cost > self.max_tokens or overflow):
                target.put(item)  # over budget: back into the queue for the next batch
                return batch
            batch.append(item)

    def run_batch(self, batch: List[WorkItem]):
        """One generate() call for the whole batch; results go back per item
        (interactive_hosted.py:119-172).  A RuntimeError (device fault) propagates, any other
        exception is reported to every caller of the batch."""
        request = {"inputs": [], "min_tokens": [], "max_tokens": []}
        for item in batch:
            ro = item.data
            request["inputs"].append(ro["input"])
            request["min_tokens"].append(ro.get("min_tokens", 0))
            request["max_tokens"].append(ro.get("max_tokens", self.max_seq_len))
            for key in SHARED_ARGS:  # assumption of the reference: the batch agrees on these
                if key in ro:
                    request[key] = ro[key]
        request["seed"] = self._rng.randint(1, 20000)
        try:
            generations = self.generator.generate(**request)
        except RuntimeError:
            raise
        except Exception as e:  # noqa: BLE001 - reported to the callers, as in the reference
            generations = [e] * len(batch)
        for item, gen in zip(batch, generations):
            item.return_queue.put((item.uid, gen))

    def step(self) -> int:
        """Collects and runs at most one batch; returns its size."""
        batch = self.collect_batch()
        if batch:
            self.run_batch(batch)
        return len(batch)

    def serve_forever(self):
        while not self._stop.is_set():
            if self.step() == 0:
                self._stop.wait(self.timeout)

    def stop(self):
        self._stop.set()
