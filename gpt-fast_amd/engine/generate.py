"""The generation loop: prompts in, new tokens out (reference generate.py:59-83, 139-211).

A batch of requests starts together: all prompts, of unequal length, go through one
prefill step, which yields each request's first new token; then every step brings one
token per live request.  A request ends when it has ``max_new_tokens`` new tokens or
draws a stop token (kept as its last token); its slot goes back to the cache at once
and the others go on.  More requests than fit in one batch run as batches one after
another.  The reference generates for one prompt repeated over the batch, always
``max_new_tokens`` tokens, with no stop condition (generate.py:174-176, 205).

The loop's decisions live in :class:`BatchRun`, which knows nothing of devices: it is
driven through a *stepper* with ``start_sequence()``, ``end_sequence(slot)`` and
``next_tokens(entries) -> list of int``.
"""
import time
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

from ..sampling import SamplingParams
from .batch import Entry


@dataclass
class GenerationResult:
    tokens: List[List[int]]                 # new tokens of each request, in request order
    finish_reasons: List[str]               # "stop" or "length"
    stats: Dict[str, float] = field(default_factory=dict)

    def sequences(self, prompts: Sequence[Sequence[int]]) -> List[List[int]]:
        return [list(p) + t for p, t in zip(prompts, self.tokens)]


class BatchRun:
    """One batch from prefill to its last token."""

    def __init__(self, stepper, prompts: Sequence[Sequence[int]], keys: Sequence[int],
                 max_new_tokens: int, stop_tokens=(), callback: Optional[Callable] = None):
        if max_new_tokens < 1:
            raise ValueError("max_new_tokens must be at least 1")
        for p in prompts:
            if len(p) == 0:
                raise ValueError("a prompt needs at least one token")
        self.stepper = stepper
        self.prompts = [list(p) for p in prompts]
        self.keys = list(keys)
        self.max_new = max_new_tokens
        self.stop = frozenset(int(t) for t in stop_tokens)
        self.callback = callback
        self.new: List[List[int]] = [[] for _ in prompts]
        self.reason: List[Optional[str]] = [None] * len(prompts)
        self.slots: List[Optional[int]] = [None] * len(prompts)
        self.steps = 0

    def live(self) -> List[int]:
        return [i for i, r in enumerate(self.reason) if r is None]

    def _take(self, rows: List[int], tokens: Sequence[int]) -> None:
        """Record one drawn token per live row and end the rows that are done."""
        for i, t in zip(rows, tokens):
            t = int(t)
            self.new[i].append(t)
            if t in self.stop:
                self.reason[i] = "stop"
            elif len(self.new[i]) >= self.max_new:
                self.reason[i] = "length"
            if self.reason[i] is not None:
                self.stepper.end_sequence(self.slots[i])
                self.slots[i] = None
        if self.callback is not None:
            self.callback(rows, [int(t) for t in tokens])

    def _decode_in_session(self) -> None:
        """One-token steps through a session that keeps the drawn tokens on the device.
        A step is launched before the tokens of the step before it are read, so a stop
        token is noticed one step late; what that step drew for the ended request is
        dropped.  Requests that end by length are known beforehand and are not launched."""
        rows = self.live()
        session = self.stepper.open_session(
            [self.slots[i] for i in rows], [self.keys[i] for i in rows],
            [self.new[i][-1] for i in rows], self.max_new - 1)
        launched = {i: len(self.new[i]) for i in rows}       # tokens drawn or under way
        pending = None
        try:
            self._drive(session, rows, launched, pending)
        finally:
            session.close()

    def _drive(self, session, rows, launched, pending) -> None:
        while True:
            active = [i for i in rows if self.reason[i] is None and launched[i] < self.max_new]
            handle = None
            if active:
                for r, i in enumerate(rows):
                    if self.reason[i] is not None and session.slots[r] is not None:
                        session.retire(r)
                handle = (active, session.launch())
                for i in active:
                    launched[i] += 1
                self.steps += 1
            if pending is not None:
                was_active, h = pending
                tokens = session.collect(h)
                keep = [i for i in was_active if self.reason[i] is None]
                self._take(keep, [tokens[rows.index(i)] for i in keep])
            pending = handle
            if pending is None:
                break

    def run(self):
        try:
            for i in range(len(self.prompts)):
                self.slots[i] = self.stepper.start_sequence()
            rows = self.live()
            entries = [Entry(self.slots[i], self.prompts[i], want=[len(self.prompts[i]) - 1],
                             key=self.keys[i]) for i in rows]
            self._take(rows, self.stepper.next_tokens(entries))       # generate.py:180
            self.steps = 1
            if self.live() and hasattr(self.stepper, "open_session"):
                self._decode_in_session()
            while True:
                rows = self.live()
                if not rows:
                    break
                entries = [Entry(self.slots[i], [self.new[i][-1]], want=[0], key=self.keys[i])
                           for i in rows]
                self._take(rows, self.stepper.next_tokens(entries))   # generate.py:72-81
                self.steps += 1
        finally:
            for i, s in enumerate(self.slots):
                if s is not None:
                    self.stepper.end_sequence(s)
                    self.slots[i] = None
        return self.new, self.reason


class EngineStepper:
    """Drives an :class:`~.step.Engine` and a sampler for :class:`BatchRun`."""

    def __init__(self, engine, params: SamplingParams, use_graph: bool = True):
        self.engine = engine
        self.params = params
        self.use_graph = use_graph
        self.prefill_seconds = 0.0
        self.decode_seconds = 0.0
        self.decode_steps = 0

    def start_sequence(self) -> int:
        return self.engine.start_sequence()

    def end_sequence(self, slot: int) -> None:
        self.engine.end_sequence(slot)

    def next_tokens(self, entries):
        import torch
        from ..sampling import sample
        t0 = time.perf_counter()
        batch = self.engine.prepare(entries)
        logits = self.engine.model.forward(batch, self.engine.cache)
        # the drawn token sits one place after the last token of each entry
        tokens = sample(logits, self.params, batch.row_keys, batch.want_pos, position_offset=1)
        out = tokens.tolist()
        dt = time.perf_counter() - t0
        if batch.is_decode:
            self.decode_seconds += dt
            self.decode_steps += 1
        else:
            self.prefill_seconds += dt
        return out


    def open_session(self, slots, keys, last_tokens, max_new_tokens):
        import torch
        from .decode import DecodeSession
        first = torch.tensor(list(last_tokens), dtype=torch.int32, device=self.engine.rt.device)
        return _TimedSession(DecodeSession(self.engine, slots, keys, first, self.params,
                                           use_graph=self.use_graph,
                                           max_new_tokens=max_new_tokens), self)


class _TimedSession:
    """A decode session that books its time to the stepper's counters."""

    def __init__(self, session, stepper):
        self.session = session
        self.stepper = stepper
        self.t_last = None

    @property
    def slots(self):
        return self.session.slots

    def retire(self, row):
        self.session.retire(row)

    def close(self):
        self.session.close()

    def launch(self):
        if self.t_last is None:
            self.t_last = time.perf_counter()
        return self.session.launch()

    def collect(self, handle):
        out = self.session.collect(handle)
        now = time.perf_counter()
        self.stepper.decode_seconds += now - self.t_last
        self.stepper.decode_steps += 1
        self.t_last = now
        return out


def split_batches(n_requests: int, batch_size: Optional[int]) -> List[List[int]]:
    if batch_size is None or batch_size >= n_requests:
        return [list(range(n_requests))] if n_requests else []
    if batch_size < 1:
        raise ValueError("batch_size must be at least 1")
    return [list(range(i, min(i + batch_size, n_requests)))
            for i in range(0, n_requests, batch_size)]


def require_room(engine, prompts, max_new_tokens: int, batches) -> None:
    """Before anything runs: every request stays within the model's positions (the
    reference clamps its cache to them, generate.py:160-163) and every batch fits the cache
    when all its requests have grown to their full length (the last token drawn is never
    fed, so a request caches ``prompt + max_new_tokens - 1`` tokens)."""
    plan = getattr(getattr(engine, "model", None), "plan", None)
    most = getattr(plan, "max_positions", None)
    for i, p in enumerate(prompts):
        if most is not None and len(p) + max_new_tokens > most:
            raise ValueError(f"request {i}: a prompt of {len(p)} tokens and {max_new_tokens} new "
                             f"ones exceed the model's {most} positions")
    cache = getattr(engine, "cache", None)
    if cache is None:
        return
    for rows in batches:
        cache.require_room([len(prompts[i]) + max_new_tokens - 1 for i in rows])


def generate(engine, prompts: Sequence[Sequence[int]], max_new_tokens: int, *,
             temperature: float = 0.8, top_k: Optional[int] = None,
             stop_tokens: Optional[Sequence[int]] = None, seed: int = 1234,
             batch_size: Optional[int] = None, callback: Optional[Callable] = None,
             use_graph: bool = True, stepper=None) -> GenerationResult:
    """Generate up to ``max_new_tokens`` tokens for every prompt (lists of token ids).

    ``temperature`` and ``top_k`` mean what they mean in the reference's ``generate``
    (generate.py:44-57); ``temperature=0`` is greedy.  ``stop_tokens`` defaults to the
    model's end-of-sequence ids (none if the configuration names none).  ``batch_size``
    bounds how many requests run together; the rest follow in further batches.
    ``use_graph`` replays the one-token step as a captured HIP graph.
    ``callback(rows, tokens)`` is called after every step with the indices of the
    requests that drew a token and the tokens (the reference calls back per step too,
    generate.py:79)."""
    params = SamplingParams(temperature=temperature, top_k=top_k, seed=seed)
    if stop_tokens is None:
        stop_tokens = engine.model.plan.stop_tokens
    stepper = stepper or EngineStepper(engine, params, use_graph=use_graph)
    batches = split_batches(len(prompts), batch_size)
    require_room(engine, prompts, max_new_tokens, batches)
    tokens: List[List[int]] = [[] for _ in prompts]
    reasons: List[str] = ["length"] * len(prompts)
    steps = 0
    t0 = time.perf_counter()
    for rows in batches:
        cb = None
        if callback is not None:
            cb = (lambda r, t, rows=rows: callback([rows[i] for i in r], t))
        run = BatchRun(stepper, [prompts[i] for i in rows], rows, max_new_tokens, stop_tokens, cb)
        new, why = run.run()
        steps += run.steps
        for i, n, w in zip(rows, new, why):
            tokens[i], reasons[i] = n, w
    stats = {"seconds": time.perf_counter() - t0, "steps": steps,
             "new_tokens": sum(len(t) for t in tokens)}
    for k in ("prefill_seconds", "decode_seconds", "decode_steps"):
        if hasattr(stepper, k):
            stats[k] = getattr(stepper, k)
    return GenerationResult(tokens, reasons, stats)
