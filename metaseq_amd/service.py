"""Serving loops in front of ``GeneratorInterface``, without a web layer.

Two engines share one front (``submit`` from any thread, ``step`` / ``serve_forever`` on the one
thread that drives the GPU, results delivered through a per-request queue):

* ``BatchingService`` - run-to-completion batches, the policy of the reference's hosted service
  (metaseq/cli/interactive_hosted.py:66-175 with metaseq/service/queue.py and workers.py):
  requests wait in one backlog per sampling signature, the fullest backlog is served cheapest
  request first, and a batch - a padded rectangle - closes when one more request would push
  ``longest cost x rows`` over the token budget or ``longest prompt + longest continuation`` over
  the sequence length, or when nothing arrives for ``timeout_ms``.
* ``ContinuousBatcher`` - no reference counterpart: a fixed set of slots over one KV cache with
  per-row lengths; a request is prefilled into a free slot whenever one exists and leaves it the
  moment it ends, while the other rows keep decoding.  Greedy and sampled requests share the
  batch; each row follows its own temperature, nucleus (fixed or decaying), repetition
  penalties and ``min_tokens`` / ``max_tokens`` / end-of-sequence rules, and gets the record a
  single-request ``GeneratorInterface.generate`` call would give it, alternatives per position
  (``logprobs``) included.
"""
import heapq
import itertools
import math
import queue
import random
import threading
from typing import Any, Dict, List, Optional


def upload(values, dtype, device):
    """A short host list as a device tensor, stream-ordered through pinned memory (see
    ``transformer_decoder.upload``): the serving loop must not wait for the step in flight
    every time it hands the GPU a few indices."""
    from .transformer_decoder import upload as _upload
    return _upload(values, dtype, device)

# options that must agree within a run-to-completion batch (metaseq/service/workers.py:13-23)
SIGNATURE_OPTIONS = ("temperature", "top_p", "n", "lambda_decay", "omega_bound", "alpha_presence",
                     "alpha_frequency", "alpha_presence_src", "alpha_frequency_src")
# options handed through to generate() from the requests of a batch
# (interactive_hosted.py:125-142)
CALL_OPTIONS = ("temperature", "top_p", "n", "best_of", "echo", "logprobs", "stop", "omega_bound",
                "lambda_decay", "alpha_presence", "alpha_frequency", "alpha_presence_src",
                "alpha_frequency_src", "alpha_src_penalty_end_idx")
MAX_SEQ_LEN = 2048        # metaseq/service/constants.py:8
MAX_BATCH_TOKENS = 3072   # metaseq/service/constants.py:10


def prompt_cost(n_tokens: int) -> int:
    """Work estimate of a prompt: linear layers plus attention
    (metaseq/service/workers.py:57-59)."""
    return n_tokens + int(math.ceil((n_tokens / 10) ** 2))


class Request:
    """One prompt with its generation options and the queue its answer goes to."""

    __slots__ = ("uid", "prompt", "options", "reply", "cost")

    def __init__(self, uid: int, prompt: List[int], options: Dict[str, Any]):
        self.uid = uid
        self.prompt = list(prompt)
        self.options = dict(options)
        self.reply: "queue.Queue" = queue.Queue()
        self.cost = prompt_cost(len(self.prompt))

    @property
    def new_tokens(self) -> int:
        return int(self.options.get("max_tokens", 0) or 0)

    @property
    def signature(self) -> str:
        return "|".join("%s=%s" % (k, self.options.get(k)) for k in sorted(SIGNATURE_OPTIONS))

    @property
    def rank(self):
        """Cheapest first, earlier submission first among equals (workers.py:26-50)."""
        return (self.cost, self.uid)

    def answer(self, result):
        self.reply.put((self.uid, result))


class Backlog:
    """Waiting requests, one heap per signature, behind one condition variable."""

    def __init__(self):
        self._heaps: Dict[str, list] = {}
        self._cv = threading.Condition()

    def put(self, req: Request, signature: Optional[str] = None):
        with self._cv:
            heap = self._heaps.setdefault(req.signature if signature is None else signature, [])
            heapq.heappush(heap, (req.rank, req))
            self._cv.notify_all()

    def __len__(self):
        with self._cv:
            return sum(len(h) for h in self._heaps.values())

    def fullest(self) -> Optional[str]:
        with self._cv:
            live = [(len(h), k) for k, h in self._heaps.items() if h]
            if not live:
                return None
            return max(live, key=lambda e: e[0])[1]

    def take_oldest(self, signature: str, due) -> Optional[Request]:
        """The earliest-submitted request of one signature if ``due(request)`` holds, else
        None (the request stays where it is)."""
        with self._cv:
            heap = self._heaps.get(signature) or []
            if not heap:
                return None
            i = min(range(len(heap)), key=lambda j: heap[j][1].uid)
            req = heap[i][1]
            if not due(req):
                return None
            heap[i] = heap[-1]
            heap.pop()
            heapq.heapify(heap)
            return req

    def take(self, signature: str, wait: float = 0.0) -> Optional[Request]:
        """Cheapest request of one signature; waits up to ``wait`` seconds for one to arrive."""
        with self._cv:
            heap = self._heaps.setdefault(signature, [])
            if not heap and wait > 0:
                self._cv.wait_for(lambda: bool(heap), timeout=wait)
            return heapq.heappop(heap)[1] if heap else None


class Rectangle:
    """A run-to-completion batch: rows padded to the longest member.  It owns the arithmetic
    that decides whether one more request still fits."""

    def __init__(self, token_budget: int, max_seq_len: int):
        self.token_budget, self.max_seq_len = token_budget, max_seq_len
        self.members: List[Request] = []
        self._widest = self._longest_prompt = self._longest_new = 0

    def fits(self, req: Request) -> bool:
        if not self.members:
            return True  # a lone request is never refused here; generate() judges it
        padded = max(self._widest, req.cost) * (len(self.members) + 1)
        span = max(self._longest_prompt, len(req.prompt)) + max(self._longest_new, req.new_tokens)
        return padded <= self.token_budget and span <= self.max_seq_len

    def add(self, req: Request):
        self.members.append(req)
        self._widest = max(self._widest, req.cost)
        self._longest_prompt = max(self._longest_prompt, len(req.prompt))
        self._longest_new = max(self._longest_new, req.new_tokens)

    def call_arguments(self, seed: int) -> Dict[str, Any]:
        args: Dict[str, Any] = {
            "inputs": [r.prompt for r in self.members],
            "min_tokens": [r.options.get("min_tokens", 0) for r in self.members],
            "max_tokens": [r.options.get("max_tokens", self.max_seq_len) for r in self.members],
            "seed": seed,
        }
        for r in self.members:  # members share a signature; later ones win on the rest
            args.update({k: r.options[k] for k in CALL_OPTIONS if k in r.options})
        return args

    def answer(self, results):
        for req, res in zip(self.members, results):
            req.answer(res)


class _Front:
    """What both engines share: request numbering, the blocking call, the serving loop."""

    def __init__(self, idle_wait: float):
        self._uids = itertools.count()
        self._uid_lock = threading.Lock()
        self._halt = threading.Event()
        self._idle_wait = idle_wait

    def _new_request(self, prompt, options) -> Request:
        with self._uid_lock:
            uid = next(self._uids)
        return Request(uid, prompt, options)

    def generate(self, encoded_prompt: List[int], **options):
        """Blocking convenience call; needs ``serve_forever`` running on another thread."""
        _, result = self.submit(encoded_prompt, **options).get()
        if isinstance(result, Exception):
            raise result
        return result

    def serve_forever(self):
        try:
            while not self._halt.is_set():
                if self.step() == 0:
                    self._halt.wait(self._idle_wait)
        finally:
            self._flush()   # answers an engine may hold back until its next step

    def _flush(self):
        pass

    def stop(self):
        self._halt.set()


class BatchingService(_Front):
    """Run-to-completion batching in front of anything with ``generate(inputs=..., ...)``."""

    def __init__(self, generator, max_tokens: int = MAX_BATCH_TOKENS,
                 max_seq_len: int = MAX_SEQ_LEN, timeout_ms: float = 100.0, seed: int = None):
        super().__init__(timeout_ms / 1000.0)
        self.generator = generator
        self.max_tokens, self.max_seq_len = max_tokens, max_seq_len
        self.timeout = timeout_ms / 1000.0
        self.backlog = Backlog()
        self._rng = random.Random(seed)

    def submit(self, encoded_prompt: List[int], **options) -> "queue.Queue":
        """Queues one prompt; the returned queue receives ``(uid, result_or_exception)``."""
        req = self._new_request(encoded_prompt, options)
        self.backlog.put(req)
        return req.reply

    def plan(self) -> Rectangle:
        """The next batch: cheapest-first from the fullest backlog until one more would not fit
        or nothing arrives within the timeout."""
        batch = Rectangle(self.max_tokens, self.max_seq_len)
        signature = self.backlog.fullest()
        while signature is not None:
            req = self.backlog.take(signature, wait=self.timeout)
            if req is None:
                break
            if not batch.fits(req):
                self.backlog.put(req)  # opens the next batch
                break
            batch.add(req)
        return batch

    def run(self, batch: Rectangle):
        """One generate() call for the batch.  A RuntimeError is a device fault and propagates
        (the reference's worker dies on it and is restarted, interactive_hosted.py:161-171);
        any other exception is the answer every member gets."""
        try:
            results = self.generator.generate(
                **batch.call_arguments(self._rng.randint(1, 20000)))
        except RuntimeError:
            raise
        except Exception as e:  # noqa: BLE001 - delivered to the callers
            results = [e] * len(batch.members)
        batch.answer(results)

    def step(self) -> int:
        """Plans and runs at most one batch; returns its size."""
        batch = self.plan()
        if batch.members:
            self.run(batch)
        return len(batch.members)


class _Row:
    """One replica of a request while it occupies a slot."""

    __slots__ = ("group", "replica", "tokens", "scores", "n_new", "min_new", "max_new", "last",
                 "done", "top", "released")

    def __init__(self, group: "_Group", replica: int, tokens: List[int], scores: List[float]):
        req = group.req
        self.group, self.replica = group, replica
        self.tokens, self.scores = tokens, scores
        self.n_new = 0
        self.min_new = int(req.options.get("min_tokens", 0) or 0)
        self.max_new = group.max_new
        self.last = tokens[-1]
        self.done = False
        self.released = False   # the device has been told to drop the row (its slot is still ours)
        # with ``logprobs``: per position of ``tokens``, the most likely ids and their
        # log-probabilities ((values, ids) lists; empty lists where nothing was predicted)
        self.top: Optional[List[tuple]] = None

    def mode(self, ahead: int = 0) -> int:
        """Selection regime of this row's next token (``ahead``: tokens chosen on the device
        that the host has not seen yet): end-of-sequence and stop tokens are barred until
        ``min_tokens`` are out, and the last allowed token can only be end-of-sequence, as in
        the generation loop (metaseq/sequence_generator.py:272-284)."""
        n, m = self.n_new + ahead, 0
        if n < self.min_new:
            m |= 1  # MSA_ROW_BAN_EARLY
        if n >= self.max_new - 1:
            m |= 2  # MSA_ROW_ONLY_EOS
        return m

    def take(self, token: int, score: float, eos: int, stop) -> bool:
        """Records the chosen token; True when the row has ended."""
        self.tokens.append(token)
        self.scores.append(score)
        self.n_new += 1
        self.last = token
        self.done = token == eos or token in stop or self.n_new >= self.max_new
        return self.done


class _Launched:
    """A decode step that has been queued: which result buffer it writes, the rows it steps
    (by slot), and the alternatives of the rows that record them."""

    def __init__(self, buf: int, rows: Dict[int, "_Row"]):
        self.buf, self.rows = buf, rows
        self.watched, self.top = None, None


class _Group:
    """A request in flight: its replicas (``best_of`` rows that share the prompt), how they are
    chosen, and the records of those that have ended."""

    def __init__(self, req: Request, max_new: int):
        o = req.options
        self.req, self.max_new = req, max_new
        self.n = int(o.get("n", 1) or 1)
        self.replicas = int(o.get("best_of") or self.n)
        # the reference's reading of the two options (metaseq/hub_utils.py:262-274): top_p <= 0
        # or temperature 0 mean greedy; temperature 0 also means "do not scale"
        temperature = o.get("temperature", 1.0)
        temperature = 1.0 if temperature is None else float(temperature)
        top_p = o.get("top_p", -1.0)
        top_p = float(top_p) if (top_p is not None and top_p > 0) else 0.0
        if temperature == 0:
            temperature, top_p = 1.0, 0.0
        self.temperature, self.topp = temperature, top_p

        def weight(key):
            return max(0.0, float(o.get(key, 0.0) or 0.0))
        # repetition penalties (metaseq/sequence_generator.py:118-123, 478-534): presence,
        # frequency, and the same two for the prompt's tokens
        self.alphas = (weight("alpha_presence"), weight("alpha_frequency"),
                       weight("alpha_presence_src"), weight("alpha_frequency_src"))
        self.src_end = int(o.get("alpha_src_penalty_end_idx", -1) or -1)
        self.penalised = max(self.alphas) > 0
        # factual nucleus (:107-116, 443-476): only a sampled row has a nucleus to decay
        decay = o.get("lambda_decay", -1)
        self.decay = float(decay) if (decay is not None and decay > 0 and top_p > 0) else -1.0
        omega = o.get("omega_bound", 0.3)
        self.omega = float(0.3 if omega is None else omega)
        self.logprobs = int(o.get("logprobs", 0) or 0)
        # rows chosen inside the vocabulary projection (greedy on the unscaled logits) or by the
        # sampling kernel on the stored logits (any other temperature, nucleus sampling,
        # penalties, recorded distributions)
        self.plain = (temperature == 1.0 and top_p == 0.0 and not self.penalised
                      and self.logprobs == 0)
        self.finished: Dict[int, "_Row"] = {}


class SlotBatch:
    """The running batch of the continuous engine: which request sits in which slot, and the
    arithmetic that decides whether a request can be taken in."""

    def __init__(self, slots: int, capacity: int):
        self.capacity = capacity
        self.rows: List[Optional[_Row]] = [None] * slots

    def free_slot(self) -> Optional[int]:
        for i, r in enumerate(self.rows):
            if r is None:
                return i
        return None

    def free_slots(self) -> List[int]:
        return [i for i, r in enumerate(self.rows) if r is None]

    def active(self):
        return [(i, r) for i, r in enumerate(self.rows) if r is not None]

    def room_for(self, req: Request) -> int:
        """New tokens the request may generate in a slot: its own limit, capped by what the
        slot's cache holds after the prompt and its leading end-of-sequence token (0: the
        prompt itself does not fit)."""
        left = self.capacity - (len(req.prompt) + 1)
        if left < 1:
            return 0
        asked = req.new_tokens or left
        return max(1, min(asked, left))


class ContinuousBatcher(_Front):
    """Continuous batching over ``slots`` rows of one KV cache.

    ``interface`` is the ``GeneratorInterface`` whose model, dictionary and tokenizer are used;
    ``capacity`` is the number of positions a slot can hold (prompt + continuation).  Greedy and
    sampled requests (``temperature``, ``top_p``) share the running batch, each row under its own
    temperature, nucleus and length rules; ``n`` / ``best_of`` replicas of a request are rows of
    their own that share one prefill.  Repetition penalties and the factual-nucleus decay are
    per-row state of the sampling kernel's call; with ``logprobs`` the kernel also stores the
    step's masked log-probabilities, of which the requested number of best entries is kept per
    position.

    ``noise_fn(request, replica, position, vocab)`` -> fp32 [vocab] device tensor, if given,
    supplies the Exp(1) numbers of the draw that chooses the token at ``position`` of that
    replica (tests hand both engines the same numbers); otherwise they come from torch's device
    generator.  A request that has waited ``patience`` steps is served before cheaper ones.

    ``prefill_batch`` > 1 lets up to that many waiting requests share one prefill (the weights
    are read once for all their prompts; a lone short prompt's prefill costs a third to a half
    of a full batch's decode step), and ``prefill_wait`` holds fewer waiting requests back for up
    to that many steps while rows are decoding, for company.  With the default (1, 0) every
    request is prefilled alone and its result does not depend on its neighbours to the last
    bit; a shared prefill runs on other tile shapes, so results can then differ in the last bit
    of a logit, as they do between batches of the reference's own service."""

    def __init__(self, interface, slots: int = 32, capacity: int = MAX_SEQ_LEN,
                 idle_ms: float = 2.0, noise_fn=None, patience: int = 64,
                 prefill_batch: int = 1, prefill_wait: int = 0):
        super().__init__(idle_ms / 1000.0)
        import torch

        from . import _capi
        self._torch, self._capi = torch, _capi
        self.interface = interface
        self.model = interface.models[0]
        self.decoder = self.model.decoder
        self.dict = interface.tgt_dict
        self.device = interface.device
        capacity = min(int(capacity), self.decoder.max_positions())
        self.batch = SlotBatch(slots, capacity)
        self.backlog = Backlog()
        self.cache = None  # allocated with the first request
        self._stop: tuple = ()  # stop ids of the running batch
        self.noise_fn, self.patience = noise_fn, int(patience)
        self.prefill_batch, self.prefill_wait = max(1, int(prefill_batch)), int(prefill_wait)
        # with rows running, queue the decode step before the admissions of the same call
        self.launch_before_admission = True
        self._held = 0          # steps the waiting requests have been held back for company
        self._done: List[_Group] = []   # ended requests whose records are not built yet
        dev = self.device
        # What a step uploads - every slot's last token (int64), temperature (fp32), row mode
        # and row mode for the sampling kernel (uint8) - lies in one pinned staging buffer and
        # goes to the device in one copy that nothing waits for (four tensors built from lists
        # cost four blocking copies, 0.2 ms each, while the GPU sits idle between two steps).
        n = slots
        on_gpu = torch.device(dev).type == "cuda"
        self._stage_host = torch.zeros(15 * n + 8, dtype=torch.uint8, pin_memory=on_gpu)
        self._stage_dev = torch.zeros(15 * n + 8, dtype=torch.uint8, device=dev)
        view = lambda buf: (buf[:8 * n].view(torch.long), buf[8 * n:12 * n].view(torch.float32),
                            buf[12 * n:13 * n], buf[13 * n:14 * n], buf[14 * n:15 * n])
        self._h_last, self._h_temp, self._h_mode, self._h_smode, self._h_fed = (
            t.numpy() for t in view(self._stage_host))
        self._last, self._temp, self._mode, self._smode, self._fed = view(self._stage_dev)
        # results of a step: two buffers (the step in flight and the one before it), each with
        # a pinned host copy that is queued right behind the step and waited for by its own event
        self._tok = torch.zeros(2, slots, dtype=torch.long, device=dev)
        self._score = torch.zeros(2, slots, dtype=torch.float32, device=dev)
        self._host_tok = torch.zeros(2, slots, dtype=torch.long, pin_memory=on_gpu)
        self._host_score = torch.zeros(2, slots, dtype=torch.float32, pin_memory=on_gpu)
        self._events = [torch.cuda.Event(), torch.cuda.Event()] if on_gpu else None
        self._inflight: Optional[_Launched] = None
        # Per-slot parameters of the rows the sampling kernel chooses, set at admission in a
        # pinned mirror and uploaded, if anything changed, with the step's first copy: initial
        # nucleus, decay factor (<= 0: none), floor ([slots, 3]) and the four penalty weights
        # ([slots, 4], contiguous: the kernel's penalty_rows).
        self._par_host = torch.zeros(7 * n, dtype=torch.float32, pin_memory=on_gpu)
        self._par_dev = torch.zeros(7 * n, dtype=torch.float32, device=dev)
        self._h_par = self._par_host[:3 * n].view(n, 3).numpy()
        self._h_pen = self._par_host[3 * n:].view(n, 4).numpy()
        self._h_par[:, 1] = -1.0
        par = self._par_dev[:3 * n].view(n, 3)
        self._initp, self._lam, self._omega = par[:, 0:1], par[:, 1:2], par[:, 2:3]
        self._pen = self._par_dev[3 * n:].view(n, 4)
        self._par_dirty = True
        # state allocated with the first request that needs it: [slots] current nucleus,
        # [slots, 1] tokens since the last full stop, [slots, V] logits, noise, token counts and
        # log-probability rows
        self._topp = self._logits = self._noise = self._since = None
        self._counts = self._counts_src = self._lprobs = None
        self._full_stop = torch.tensor([self.dict.index(w) for w in (".", "?", "!")],
                                       dtype=torch.long, device=dev)
        self._clock = 0         # step() calls so far; a request's arrival is stamped with it
        self._arrived: Dict[int, int] = {}
        self.steps = 0          # decode steps run
        self.rows_stepped = 0   # active rows summed over those steps

    # -- producer side ------------------------------------------------------------------
    def submit(self, encoded_prompt: List[int], **options) -> "queue.Queue":
        req = self._new_request(encoded_prompt, options)
        problem = self._why_not(req)
        if problem:
            req.answer(ValueError(problem))
        else:
            self._arrived[req.uid] = self._clock
            self.backlog.put(req, signature="")  # one queue: all requests can share the batch
        return req.reply

    def _why_not(self, req: Request) -> Optional[str]:
        o = req.options
        temperature = o.get("temperature", 1.0)
        if temperature is not None and temperature < 0:
            return "temperature must be >= 0"
        n, best_of = int(o.get("n", 1) or 1), int(o.get("best_of") or 0)
        if n < 1 or (best_of and best_of < n):
            return "best_of must be at least n, and n at least 1"
        if max(n, best_of) > len(self.batch.rows):
            return ("%d replicas do not fit the %d slots of the running batch"
                    % (max(n, best_of), len(self.batch.rows)))
        if (o.get("logprobs", 0) or 0) > len(self.dict):
            return "logprobs asks for more alternatives than the vocabulary has"
        decay = o.get("lambda_decay", -1)
        if (decay is not None and decay > 0 and (o.get("top_p") or 0) > 0
                and all(int(i) == self.dict.unk() for i in self._full_stop.tolist())):
            return ("factual-nucleus sampling (lambda_decay > 0) needs a dictionary that "
                    "resolves '.', '?' and '!' to token ids")
        if len(o.get("stop") or []) > 14:
            return "at most 14 stop tokens are supported"
        if self.batch.room_for(req) == 0:
            return ("a prompt of %d tokens does not fit a slot of %d positions"
                    % (len(req.prompt), self.batch.capacity))
        return None

    # -- consumer side ------------------------------------------------------------------
    def _sampling_state(self):
        """Per-slot state of the rows chosen by the sampling kernel, on first use."""
        if self._topp is None:
            torch, dev, slots = self._torch, self.device, len(self.batch.rows)
            V = len(self.dict)
            self._topp = torch.zeros(slots, dtype=torch.float32, device=dev)
            self._logits = torch.empty(slots, V, dtype=torch.float16, device=dev)
            self._noise = torch.empty(slots, V, dtype=torch.float32, device=dev)
            self._since = torch.zeros(slots, 1, dtype=torch.float32, device=dev)

    def _penalty_state(self):
        if self._counts is None:
            torch, slots, V = self._torch, len(self.batch.rows), len(self.dict)
            self._counts = torch.zeros(slots, V, dtype=torch.long, device=self.device)
            self._counts_src = torch.zeros(slots, V, dtype=torch.long, device=self.device)

    def _logprob_state(self):
        if self._lprobs is None:
            self._lprobs = self._torch.empty(len(self.batch.rows), len(self.dict),
                                             dtype=self._torch.float32, device=self.device)

    def _nucleus_now(self):
        """Every slot's nucleus for the next draw: the request's top-p, decayed by its factor
        per token since the last full stop and never below its floor (the arithmetic of
        metaseq/sequence_generator.py:443-476, in fp32 on the device)."""
        torch = self._torch
        decay = (self._since - 1).clamp_(min=0)
        decayed = torch.maximum(self._initp * self._lam ** decay, self._omega)
        return torch.where(self._lam > 0, decayed, self._initp).view(-1)

    def _count_chosen(self, slots: List[int], tokens):
        """After a draw: a full stop restarts the decay of a row's nucleus, any other token
        extends it (``tokens``: int64 device tensor, one per listed slot)."""
        torch = self._torch
        idx = upload(slots, torch.long, self.device)
        hit = (tokens.view(-1, 1) == self._full_stop.view(1, -1)).any(dim=1, keepdim=True)
        self._since[idx] = torch.where(hit, torch.zeros_like(self._since[idx]),
                                       self._since[idx] + 1)

    def _draw_noise(self, out, rows, ahead=None):
        """Exp(1) numbers for the draws of ``rows`` ((index into ``out``, row) pairs);
        ``ahead[i]``: tokens of that row the host has not seen yet (its position counts them)."""
        if self.noise_fn is None:
            out.exponential_()
            return
        V = out.shape[1]
        for i, row in rows:
            position = len(row.tokens) + (ahead.get(i, 0) if ahead else 0)
            out[i].copy_(self.noise_fn(row.group.req, row.replica, position, V))

    def _prepare(self, slots: List[int], req: Request, noise_at: int, tok_all, score_all):
        """What the admission of ``req`` into ``slots`` (its replicas' rows) hands to the
        decoder: rows, output tensors and the keyword arguments of ``admit_slot``.  The
        request's draws use rows ``noise_at`` .. of the shared noise buffer, its first tokens
        and their scores go to the same rows of ``tok_all`` / ``score_all``."""
        torch = self._torch
        eos, pad = self.dict.eos(), self.dict.pad()
        ids = [eos] + req.prompt
        group = _Group(req, self.batch.room_for(req))
        rows = [_Row(group, j, list(ids), []) for j in range(group.replicas)]
        R = len(rows)
        tok, score = tok_all[noise_at:noise_at + R], score_all[noise_at:noise_at + R]
        extra, detail, lp = {}, {}, None
        if not group.plain:
            self._sampling_state()
            noise = None
            if group.topp > 0:
                noise = self._noise[noise_at:noise_at + R]
                self._draw_noise(noise, list(enumerate(rows)))
            extra = dict(temperature=group.temperature, topp=group.topp, noise=noise)
            V = len(self.dict)
            if group.penalised:
                self._penalty_state()
                # the prompt's token counts, leading end-of-sequence token included, up to
                # alpha_src_penalty_end_idx if given (metaseq/sequence_generator.py:380-389)
                src = upload(ids if group.src_end <= 0 else ids[:group.src_end], torch.long,
                             self.device)
                counts_src = torch.zeros(R, V, dtype=torch.long, device=self.device)
                counts_src[0].scatter_add_(0, src.clamp(0, V - 1), torch.ones_like(src))
                counts_src[1:] = counts_src[0]
                extra["penalties"] = dict(
                    alphas=group.alphas, counts_src=counts_src,
                    counts=torch.zeros(R, V, dtype=torch.long, device=self.device))
            if group.logprobs > 0:
                self._logprob_state()
                lp = extra["lprobs_out"] = torch.empty(R, V, dtype=torch.float32,
                                                       device=self.device)
                if req.options.get("echo", False):
                    extra.update(prompt_topk=group.logprobs, detail=detail)
        if R > 1:
            extra["replicas"] = slots[1:]
        call = dict(slot=slots[0], tokens=upload(ids, torch.long, self.device),
                    banned=[pad], stop=self._stop, eos=eos, mode=rows[0].mode(), tok_out=tok,
                    score_out=score, **extra)
        return dict(slots=slots, req=req, group=group, rows=rows, ids=ids, tok=tok, score=score,
                    extra=extra, detail=detail, lp=lp, call=call, at=noise_at)

    def _finish(self, p, prompt_scores, toks, scs):
        """Book-keeping after the decoder has admitted a prepared request: per-slot sampling
        state, the alternatives of the first choice and of the prompt, the rows themselves
        (``toks`` / ``scs``: its replicas' first tokens and their scores, on the host)."""
        torch = self._torch
        slots, group, rows, tok, extra = p["slots"], p["group"], p["rows"], p["tok"], p["extra"]
        eos = self.dict.eos()
        if not group.plain:
            self._h_par[slots] = (group.topp, group.decay, group.omega)
            self._h_pen[slots] = group.alphas
            self._par_dirty = True
            if group.decay > 0 or group.penalised:
                idx = upload(slots, torch.long, self.device)
            if group.decay > 0:
                self._since.index_fill_(0, idx, 0.0)
                self._count_chosen(slots, tok)
            if group.penalised:
                self._counts[idx] = extra["penalties"]["counts"]
                self._counts_src[idx] = extra["penalties"]["counts_src"]
        first_top = prompt_top = None
        if group.logprobs > 0:
            values, top_ids = p["lp"].topk(group.logprobs, dim=-1)
            first_top = list(zip(values.tolist(), top_ids.tolist()))
            # nothing is predicted for the leading token; the prompt's alternatives are kept
            # only where they can be shown (echo)
            prompt_top = [([], [])] * len(p["ids"])
            if "prompt_top" in p["detail"]:
                values, top_ids = p["detail"]["prompt_top"]
                prompt_top = [([], [])] + list(zip(values.tolist(), top_ids.tolist()))
        for j, (slot, row) in enumerate(zip(slots, rows)):
            row.scores = list(prompt_scores)
            if first_top is not None:
                row.top = list(prompt_top) + [first_top[j]]
            self.batch.rows[slot] = row
            if row.take(toks[j], scs[j], eos, self._stop):
                self._retire(slot)

    def _prefill_groups(self, prepared):
        """Which prepared requests share a prefill: at most ``prefill_batch`` of them, of
        similar lengths - a shared prefill pads every prompt to its longest, so a group is
        closed when the padded rows would exceed the real ones by more than half."""
        groups, current, real = [], [], 0
        for p in sorted(prepared, key=lambda p: len(p["ids"])):
            n = len(p["ids"])
            if current and (len(current) >= self.prefill_batch
                            or (len(current) + 1) * n > 1.5 * (real + n)):
                groups.append(current)
                current, real = [], 0
            current.append(p)
            real += n
        if current:
            groups.append(current)
        return groups

    def _admit_many(self, items):
        """Admits ``items`` ((slots, request) pairs): a prefill per request or, with
        ``prefill_batch`` > 1, one shared prefill for all of them; every request's keys and
        values are copied to its replicas' slots and each replica's first token is chosen from
        the prompt's last position.  An error is the answer of every request it concerns."""
        if self.cache is None:
            self.cache = self.decoder.new_slot_cache(len(self.batch.rows), self.batch.capacity,
                                                     self.device)
        torch = self._torch
        total = sum(len(slots) for slots, _ in items)
        tok_all = torch.zeros(total, dtype=torch.long, device=self.device)
        score_all = torch.zeros(total, dtype=torch.float32, device=self.device)
        at, prepared = 0, []
        for slots, req in items:
            prepared.append(self._prepare(slots, req, at, tok_all, score_all))
            at += len(slots)
        # every group's kernels are queued before anything is read back: the prompt scores of
        # all of them, the first tokens and their scores then come in one copy each (a read per
        # request left the GPU idle between them once the prefills were done)
        lazy = {"lazy": True} if getattr(self.decoder, "lazy_admission", False) else {}
        queued = []
        for members in self._prefill_groups(prepared):
            try:
                if len(members) == 1:
                    call = dict(members[0]["call"])
                    scores = [self.decoder.admit_slot(self.cache, call.pop("slot"),
                                                      call.pop("tokens"), **call, **lazy)]
                else:
                    scores = self.decoder.admit_slots(self.cache, [p["call"] for p in members],
                                                      **lazy)
                queued.append((members, scores))
            except RuntimeError:
                raise
            except Exception as e:  # noqa: BLE001 - these requests' own answer
                for p in members:
                    for slot in p["slots"]:
                        self.batch.rows[slot] = None
                        self.decoder.release_slot(self.cache, slot)
                    p["req"].answer(e)
        if not queued:
            return
        on_device = [sc for _, scores in queued for sc in scores if torch.is_tensor(sc)]
        flat = torch.cat(on_device).tolist() if on_device else []
        toks, scs = tok_all.tolist(), score_all.tolist()
        cursor = 0
        for members, scores in queued:
            for p, sc in zip(members, scores):
                if torch.is_tensor(sc):
                    n = sc.numel()
                    sc = [0.0] + flat[cursor:cursor + n]
                    cursor += n
                elif sc is None:
                    sc = [0.0]
                a, R = p["at"], len(p["slots"])
                try:
                    self._finish(p, sc, toks[a:a + R], scs[a:a + R])
                except RuntimeError:
                    raise
                except Exception as e:  # noqa: BLE001 - this request's own answer
                    for slot in p["slots"]:
                        self.batch.rows[slot] = None
                        self.decoder.release_slot(self.cache, slot)
                    p["req"].answer(e)

    def _retire(self, slot: int):
        row = self.batch.rows[slot]
        self.batch.rows[slot] = None
        self.decoder.release_slot(self.cache, slot)
        group = row.group
        group.finished[row.replica] = row
        if len(group.finished) < group.replicas:
            return
        # the records are built (token strings, offsets, alternatives) while the GPU runs the
        # next decode step, not between two steps
        self._done.append(group)

    def _answer(self, group: "_Group"):
        req = group.req
        try:
            from .hub_utils import TopRows
            # replicas best cumulative score first (metaseq/sequence_generator.py:325-333), each
            # as the generation loop would return it: tokens up to the end, then eos
            ranked = sorted(group.finished.values(), key=lambda r: (-sum(r.scores), r.replica))
            records = []
            for r in ranked[:group.n]:
                toks, scs = list(r.tokens), list(r.scores)
                top = list(r.top) if r.top is not None else None
                if toks[-1] != self.dict.eos():
                    toks.append(self.dict.eos())
                    scs.append(0.0)
                    if top is not None:
                        top.append(([], []))
                records.append(self.interface._record(
                    toks, scs, TopRows.from_pairs(top, group.logprobs) if top else None,
                    len(req.prompt), group.max_new, bool(req.options.get("echo", False)),
                    group.logprobs))
            req.answer(records)
        except Exception as e:  # noqa: BLE001 - delivered to the caller
            req.answer(e)

    def _flush(self):
        """Answers the requests whose last replica has ended."""
        done, self._done = self._done, []
        for group in done:
            self._answer(group)

    def _next_request(self) -> Optional[Request]:
        """The cheapest waiting request, unless the oldest one has waited ``patience`` steps."""
        old = self.backlog.take_oldest(
            "", lambda r: self._clock - self._arrived.get(r.uid, self._clock) >= self.patience)
        return old if old is not None else self.backlog.take("")

    def step(self) -> int:
        """Takes waiting requests into free slots, then runs one decode step over the occupied
        slots.  Returns the number of rows that were served (admitted, stepped or read).  The rows of
        the running batch share one stop list: a request with another one waits until the batch
        has drained, and nothing is admitted past it while it waits.  The step queued by this
        call is read by the next one (after that call has queued its own): a request's answer
        follows the call that chose its last token by one or two calls."""
        torch = self._torch
        self._clock += 1
        served = 0
        free = self.batch.free_slots()
        taken: List[tuple] = []
        while free:
            req = self._next_request()
            if req is None:
                break
            need = int(req.options.get("best_of") or req.options.get("n", 1) or 1)
            stop = tuple(sorted(req.options.get("stop") or ()))
            if ((self.batch.active() or taken) and stop != self._stop) or need > len(free):
                self.backlog.put(req, signature="")
                break
            self._stop = stop
            taken.append((free[:need], req))
            free = free[need:]
        # a shared prefill is worth waiting for: while rows are decoding, fewer admissible
        # requests than prefill_batch (few free slots, or few waiting) are held back for up to
        # prefill_wait steps
        if (taken and len(taken) < self.prefill_batch and self.prefill_wait > 0
                and self.batch.active() and self._held < self.prefill_wait):
            self._held += 1
            for _, req in reversed(taken):
                self.backlog.put(req, signature="")
            taken = []
        if taken:
            self._held = 0
            for _, req in taken:
                self._arrived.pop(req.uid, None)
            served += sum(len(slots) for slots, _ in taken)
        # With rows running, the decode step below is queued before the admissions: preparing
        # a few dozen requests takes the host as long as a decode step takes the GPU, and the
        # GPU would sit idle behind the step in flight (a tenth of the time at 256 slots).  The
        # new rows then join the step after this one.  With nothing to step, admit first.
        if taken and not (self.launch_before_admission and self.batch.active()):
            self._admit_many(taken)
            taken = []
        # The step launched by the previous call is still running, or its results are still
        # unread: its rows' tokens are on the device only.  This call launches the next step
        # first - the rows that step chose tokens for are fed from the device, their modes
        # follow from the count of their tokens alone - and reads the previous step's results
        # while the new one runs.  A row whose previous token turns out to have ended it has
        # then been stepped once more: that output is dropped.  (Reading every step's tokens
        # before launching the next leaves the GPU idle for all of the host's work between
        # two steps: a fifth of the time at 128 slots.)
        before = self._inflight
        stepping = []
        for i, row in self.batch.active():
            ahead = 1 if (before is not None and before.rows.get(i) is row) else 0
            if row.n_new + ahead >= row.max_new:
                # its last token is in flight: nothing more to decode; the device may drop it
                if ahead and not row.released:
                    self.decoder.release_slot(self.cache, i)
                    row.released = True
                continue
            stepping.append((i, row, ahead))
        self._inflight = self._launch(stepping, before) if stepping else None
        if taken:
            self._admit_many(taken)
        self._flush()   # a step is queued: the GPU works while the host writes records
        if before is not None:
            self._collect(before)
            served += len(before.rows)
        if self._inflight is None:
            self._flush()
        return served + len(stepping)

    def _launch(self, stepping, before):
        """Queues one decode step for ``stepping`` ((slot, row, tokens in flight) triples) and
        the copy of its results to pinned host memory; returns what ``_collect`` needs."""
        torch = self._torch
        eos, pad = self.dict.eos(), self.dict.pad()
        slots = len(self.batch.rows)
        buf = 1 - before.buf if before is not None else 0
        last, mode, fed = [pad] * slots, [0] * slots, [0] * slots
        general = [(i, row) for i, row, _ in stepping if not row.group.plain]
        for i, row, ahead in stepping:
            mode[i] = row.mode(ahead)
            if ahead:
                fed[i] = 1          # its last token is what the previous step chose
            else:
                last[i] = row.last
        self._h_last[:] = last
        self._h_mode[:] = mode
        self._h_fed[:] = fed
        if general:
            smode, temp = [4] * slots, [1.0] * slots  # 4 = MSA_ROW_SKIP
            for i, row in general:
                smode[i], temp[i] = mode[i], row.group.temperature
            self._h_smode[:] = smode
            self._h_temp[:] = temp
        self._stage_dev.copy_(self._stage_host, non_blocking=True)
        if self._par_dirty:
            self._par_dev.copy_(self._par_host, non_blocking=True)
            self._par_dirty = False
        feed = self._last
        if before is not None and any(fed):
            feed = torch.where(self._fed.bool(), self._tok[before.buf], self._last)
        extra = {}
        if general:
            self._topp.copy_(self._nucleus_now())
            noise = None
            drawn = [(i, row) for i, row in general if row.group.topp > 0]
            if drawn:
                noise = self._noise
                ahead_of = {i: ahead for i, _, ahead in stepping}
                self._draw_noise(noise, drawn, ahead_of)
            sampled = dict(row_mode=self._smode, temperature=self._temp, topp=self._topp,
                           noise=noise)
            if any(row.group.penalised for _, row in general):
                sampled.update(penalty_rows=self._pen, counts=self._counts,
                               counts_src=self._counts_src)
            if any(row.group.logprobs > 0 for _, row in general):
                sampled["lprobs_out"] = self._lprobs
            extra = dict(logits_out=self._logits, sampled=sampled)
        tok, score = self._tok[buf], self._score[buf]
        self.decoder.decode_slots(self.cache, feed, temperature=1.0, banned=[pad],
                                  stop=self._stop, eos=eos, row_mode=self._mode,
                                  tok_out=tok, score_out=score, **extra)
        decaying = [i for i, row in general if row.group.decay > 0]
        if decaying:
            self._count_chosen(decaying, tok[upload(decaying, torch.long, self.device)])
        launched = _Launched(buf, {i: row for i, row, _ in stepping})
        watched = [(i, row) for i, row in general if row.group.logprobs > 0]
        if watched:
            k = max(row.group.logprobs for _, row in watched)
            picked = self._lprobs[upload([i for i, _ in watched], torch.long, self.device)]
            values, top_ids = picked.topk(k, dim=-1)
            launched.watched = watched
            pinned = self._events is not None
            launched.top = tuple(
                torch.empty(t.shape, dtype=t.dtype, pin_memory=pinned).copy_(t, non_blocking=True)
                for t in (values, top_ids))
        self._host_tok[buf].copy_(tok, non_blocking=True)
        self._host_score[buf].copy_(score, non_blocking=True)
        if self._events is not None:
            self._events[buf].record()
        self.steps += 1
        self.rows_stepped += len(stepping)
        return launched

    def _collect(self, launched):
        """Reads the results of a launched step (waiting for that step alone) and books them:
        tokens, scores, alternatives; rows that have ended leave their slots."""
        if self._events is not None:
            self._events[launched.buf].synchronize()
        toks = self._host_tok[launched.buf].tolist()
        scs = self._host_score[launched.buf].tolist()
        eos = self.dict.eos()
        if launched.watched:
            values, top_ids = (t.tolist() for t in launched.top)
            for (i, row), v, t in zip(launched.watched, values, top_ids):
                if not row.done:
                    row.top.append((v[:row.group.logprobs], t[:row.group.logprobs]))
        for i, row in launched.rows.items():
            if row.done:
                continue    # it had ended a step earlier: this output is not its
            if row.take(toks[i], scs[i], eos, self._stop):
                self._retire(i)
