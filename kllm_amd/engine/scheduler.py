"""Continuous batching above the step function.

Every iteration forms a fresh batch from whatever is running, as the
reference's scheduler does (engine/scheduler.go:95-237): waiting requests are
admitted first-come-first-served while batch slots are free (:141-148), the
batch is formed under a token budget (:160-189), one step runs, each request
that asked for logits gets a token, and requests finish on an end-of-sequence
id or at their token limit (:228-232) and give their pages back.

Where this scheduler decides differently, and why:

* Prompts are cut into portions.  The reference sends a prompt whole or not at
  all and rejects prompts longer than the step budget (:64-70, :164-176).
  Here decoding requests take one token each first, then prompt portions fill
  what is left of the budget: portion = min(rest of the prompt, budget left,
  chunk size).  Only a prompt's last portion asks for logits.
* When pages run out.  The reference fails a decoding request that cannot get
  a block and lets a waiting prompt keep a partial table (:178-182).  Here a
  step is planned against the free pages before it is run, and nothing is
  held that is not used: a prompt portion shrinks to the pages that are free
  (or waits), and if a decoding request cannot get its page, or no request
  can move at all, the *youngest* running request is preempted: its pages and
  slot are given back and it returns to the front of the waiting queue with
  the tokens it has generated; it is later recomputed from prompt + generated
  tokens.  A request that could not fit the pool even alone is refused at
  submit.
* One step ahead.  While every running request is decoding and nothing waits
  for a place, a step is queued before the ids of the step before it have
  reached the host: the engine feeds them to the next step on the device
  (``Engine.step_sample_ahead``), and the device does not stand still while the
  host reads ids and prepares the next batch.  The price is that an
  end-of-sequence id is seen one step late: the request has then taken one
  more step, whose token is thrown away; its pages are given back when that
  step is over.  A step with prompt portions in it is queued the same way
  where the engine takes it (``Engine.can_queue_ahead``): its decode tokens
  name the ids of the step in flight, its portions are known.  Anything else
  -- a shortage of pages, a preemption -- first settles the step in flight and
  then takes the plain path.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Dict, Hashable, List, Optional

from ..sampling import uniform
from .engine import StepEntry

PENDING = -1     # in Request.generated: a token that is sampled but has not reached the host yet


@dataclass
class Request:
    id: int
    prompt: List[int]
    max_new_tokens: int
    temperature: float = 0.0
    seed: int = 0
    on_token: Optional[Callable[[int, int], None]] = None
    generated: List[int] = field(default_factory=list)
    cursor: int = 0          # tokens of prompt + generated already in the cache
    done: bool = False
    error: Optional[str] = None
    preemptions: int = 0
    admitted_at: int = -1    # admission counter: larger = younger
    overrun: bool = False    # ended on an end-of-sequence id while one more step was in flight

    @property
    def tokens(self) -> List[int]:
        return self.generated

    def all_tokens(self) -> List[int]:
        return self.prompt + self.generated

    def pending(self) -> int:
        """Tokens not yet in the cache."""
        return len(self.prompt) + len(self.generated) - self.cursor


@dataclass
class PlannedEntry:
    request: Request
    start: int               # first token of all_tokens() in this step
    count: int
    wants_logits: bool


@dataclass
class StepPlan:
    entries: List[PlannedEntry] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)

    @property
    def tokens(self) -> int:
        return sum(e.count for e in self.entries)


class SchedulerError(ValueError):
    pass


class Scheduler:
    """``engine`` needs: ``cache`` (a CacheManager), ``step(entries)``,
    ``release(request_id)``, ``sample(logits, temperatures, uniforms)``,
    ``eos_token_ids`` and ``max_model_len``."""

    def __init__(self, engine, max_batch: Optional[int] = None,
                 max_step_tokens: Optional[int] = None, chunk_size: Optional[int] = None,
                 row_multiple: Optional[int] = None, queue_ahead: bool = True):
        self.engine = engine
        self.queue_ahead = bool(queue_ahead)     # False: every step waits for the ids of the one before
        # The reference's default batch is 8 (engine/scheduler.go:44-46).
        self.max_batch = int(max_batch) if max_batch else 8
        self.max_step_tokens = int(max_step_tokens) if max_step_tokens else 2048
        self.chunk_size = int(chunk_size) if chunk_size else self.max_step_tokens
        sized_for = getattr(getattr(engine, "options", None), "max_step_tokens", None)
        if sized_for:                        # the engine takes no larger portion of one request
            self.chunk_size = min(self.chunk_size, int(sized_for))
        # Rows of the tiles that the engine's products work on (0: none known).  A step a few
        # tokens above a multiple pays for a whole further tile of every product.
        if row_multiple is None:
            row_multiple = getattr(engine, "step_row_multiple", 0)
        self.row_multiple = int(row_multiple or 0)
        if self.max_batch <= 0 or self.max_step_tokens <= 0 or self.chunk_size <= 0 or self.row_multiple < 0:
            raise SchedulerError("batch, token budget and chunk size must be positive")
        self.waiting: deque = deque()
        self.running: List[Request] = []
        self.requests: Dict[int, Request] = {}
        self._next_id = 0
        self._admissions = 0
        self._in_flight = None   # (handle, [(request, place in generated)]) of a step queued ahead
        self.stats = {"steps": 0, "tokens": 0, "prefill_tokens": 0, "decode_tokens": 0,
                      "preemptions": 0, "max_batch_seen": 0}

    # ------------------------------------------------------------------ submit
    def _key(self, r: Request) -> Hashable:
        return ("sched", id(self), r.id)

    def submit(self, prompt: List[int], max_new_tokens: int, temperature: float = 0.0,
               seed: int = 0, on_token=None) -> int:
        """Queue a request; returns its id.  Refuses what can never run."""
        if len(prompt) == 0 or max_new_tokens <= 0:
            raise SchedulerError("empty prompt or non-positive max_new_tokens")
        total = len(prompt) + max_new_tokens
        limit = getattr(self.engine, "max_model_len", None)
        if limit is not None and total > limit:
            raise SchedulerError(
                f"prompt of {len(prompt)} tokens plus {max_new_tokens} new ones exceeds the "
                f"longest request allowed ({limit})")
        cache = self.engine.cache
        step = min(self.chunk_size, self.max_step_tokens)
        for need, pool in zip(cache.pages_for_tokens(total, step), cache.pools):
            if need > pool.num_pages:
                raise SchedulerError(
                    f"a request of {total} tokens needs {need} pages, the pool has "
                    f"{pool.num_pages}: it could not run even alone")
        r = Request(self._next_id, list(prompt), int(max_new_tokens), float(temperature), int(seed),
                    on_token)
        self._next_id += 1
        self.requests[r.id] = r
        self.waiting.append(r)
        return r.id

    # ------------------------------------------------------------------ planning
    def _admit(self):
        cache = self.engine.cache
        while self.waiting and len(self.running) < self.max_batch and cache.slots.free_slots > 0:
            r = self.waiting.popleft()
            cache.open(self._key(r))
            r.cursor = 0
            r.admitted_at = self._admissions
            self._admissions += 1
            self.running.append(r)

    def _preempt(self, r: Request):
        self.engine.release(self._key(r))
        self.running.remove(r)
        r.cursor = 0
        r.preemptions += 1
        self.stats["preemptions"] += 1
        self.waiting.appendleft(r)

    def _holds_pages(self, r: Request) -> bool:
        rc = self.engine.cache.get(self._key(r))
        return any(p >= 0 for t in rc.tables for p in t)

    def _try_plan(self):
        """(entries, blocked): a plan against the free pages, or the request
        that stands still for want of pages."""
        cache = self.engine.cache
        free = [p.free_pages for p in cache.pools]
        budget = self.max_step_tokens
        entries: List[PlannedEntry] = []

        def fits(r, n):
            need = cache.pages_needed(self._key(r), n)
            return all(a <= b for a, b in zip(need, free)), need

        # 1. one token for every request that is decoding
        for r in self.running:
            if not (r.pending() == 1 and r.generated) or budget <= 0:
                continue
            ok, need = fits(r, 1)
            if not ok:
                return [], r
            free = [b - a for a, b in zip(need, free)]
            budget -= 1
            entries.append(PlannedEntry(r, r.cursor, 1, True))
        # 2. prompt portions into what is left of the budget
        for r in self.running:
            if budget <= 0:
                break
            if r.pending() == 1 and r.generated:
                continue
            count = min(r.pending(), budget, self.chunk_size)
            ok, need = fits(r, count)
            if not ok:
                count = self._largest_fit(r, count, free)
                if count <= 0:
                    continue
                ok, need = fits(r, count)
                if not ok:
                    continue
            free = [b - a for a, b in zip(need, free)]
            budget -= count
            entries.append(PlannedEntry(r, r.cursor, count, count == r.pending()))
        if not entries and self.running:
            return [], min(self.running, key=lambda q: q.admitted_at)
        self._trim_to_tiles(entries)
        return entries, None

    def _trim_to_tiles(self, entries: List[PlannedEntry]) -> None:
        """A step of more than one tile of rows that ends less than half a tile
        above a multiple gives the excess back from its last prompt portions:
        the tokens go into the next step, and this one does not pay a further tile
        of every product for them (512 + 31 tokens on tiles of 128: five tiles
        for 4.2 tiles' worth)."""
        m = self.row_multiple
        if not m or not entries:
            return
        total = sum(e.count for e in entries)
        excess = total % m
        if total <= m or 2 * excess >= m:
            return
        while excess and entries:
            last = entries[-1]
            if last.count == 1 and last.request.generated:
                return                                   # decoding requests are never put off
            if last.count > excess:
                last.count -= excess
                last.wants_logits = False
                return
            excess -= last.count                         # a portion smaller than the excess waits whole
            entries.pop()

    def plan(self) -> StepPlan:
        """Decide the next step.  Changes the queues (admission, preemption)
        but reserves nothing: the plan is made against the free pages."""
        plan = StepPlan()
        self._admit()
        while True:
            entries, blocked = self._try_plan()
            if blocked is None:
                plan.entries = entries
                return plan
            holders = [q for q in self.running if self._holds_pages(q)]
            victim = max(holders, key=lambda q: q.admitted_at) if holders else None
            if victim is None or (victim is blocked and len(holders) == 1):
                # No one to take pages from: the pool is held from outside this scheduler.
                blocked.done, blocked.error = True, "no pages can be freed for this request"
                self.engine.release(self._key(blocked))
                self.running.remove(blocked)
                if not self.running:
                    return plan
                continue
            self._preempt(victim)
            plan.preempted.append(victim)

    def _largest_fit(self, r: Request, count: int, free: List[int]) -> int:
        """Largest portion below ``count`` that the free pages can hold."""
        cache = self.engine.cache
        rc = cache.get(self._key(r))
        best = count - 1
        for g, grp in enumerate(cache.groups):
            room = len(rc.tables[g]) * grp.page_size - (rc.length + rc.reserved)
            best = min(best, room + free[g] * grp.page_size)
        return max(best, 0)

    # ------------------------------------------------------------------ running
    def step(self) -> List[tuple]:
        """One iteration: plan, run, sample, finish.  Returns the
        (request id, token) pairs produced."""
        ahead = self._decode_batch_ahead() if self.queue_ahead else None
        if ahead is not None:
            return self._queue_ahead(ahead)
        planned = self._plan_ahead() if self.queue_ahead else None
        if planned is not None:
            return self._queue_plan(planned)
        produced = self._settle()                # nothing is in flight below this line
        plan = self.plan()
        if not plan.entries:
            return produced
        entries = []
        for pe in plan.entries:
            toks = pe.request.all_tokens()[pe.start:pe.start + pe.count]
            entries.append(StepEntry(self._key(pe.request), toks,
                                     [pe.count - 1] if pe.wants_logits else []))
        wanting = [pe for pe in plan.entries if pe.wants_logits]
        temps = [pe.request.temperature for pe in wanting]
        us = [uniform(pe.request.seed, len(pe.request.generated)) for pe in wanting]
        try:
            if hasattr(self.engine, "step_sample"):
                toks = self.engine.step_sample(entries, temps, us)
            else:
                logits = self.engine.step(entries)
                toks = self.engine.sample(logits, temps, us) if wanting else []
        except Exception as exc:  # a failed forward fails every request of the step
            for pe in plan.entries:  # (engine/scheduler.go:197-203)
                r = pe.request
                r.done, r.error = True, f"step failed: {exc}"
                if self._key(r) in self.engine.cache:
                    self.engine.release(self._key(r))
                if r in self.running:
                    self.running.remove(r)
            raise
        self.stats["steps"] += 1
        self.stats["tokens"] += plan.tokens
        self.stats["max_batch_seen"] = max(self.stats["max_batch_seen"], len(entries))
        for pe in plan.entries:
            pe.request.cursor += pe.count
            key = "decode_tokens" if (pe.count == 1 and pe.request.generated) else "prefill_tokens"
            self.stats[key] += pe.count
        if wanting:
            eos = set(getattr(self.engine, "eos_token_ids", ()) or ())
            for pe, tok in zip(wanting, toks):
                r = pe.request
                r.generated.append(int(tok))
                produced.append((r.id, int(tok)))
                if r.on_token is not None:
                    r.on_token(r.id, int(tok))
                if int(tok) in eos or len(r.generated) >= r.max_new_tokens:
                    r.done = True
                    self.engine.release(self._key(r))
                    self.running.remove(r)
        return produced

    # ------------------------------------------------------------------ one step ahead
    def _decode_batch_ahead(self):
        """The running requests, if the next step is one decode token for each
        of them and can be queued without any decision: nothing to admit,
        nothing to cut, pages for all.  Looks, changes nothing."""
        eng = self.engine
        if not hasattr(eng, "step_sample_ahead") or not self.running:
            return None
        if self.waiting and len(self.running) < self.max_batch:
            return None
        if len(self.running) > self.max_step_tokens:
            return None
        free = [p.free_pages for p in eng.cache.pools]
        for r in self.running:
            if not (r.pending() == 1 and r.generated):
                return None
            need = eng.cache.pages_needed(self._key(r), 1)
            if any(a > b for a, b in zip(need, free)):
                return None
            free = [b - a for a, b in zip(need, free)]
        entries = [StepEntry(self._key(r), [0], [0]) for r in self.running]
        return list(self.running) if eng.can_sample_ahead(entries) else None

    def _plan_ahead(self):
        """The next step's plan, if it can be queued behind the step in flight without
        a decision that needs that step's ids: no request stands still for want of pages
        (no preemption), every token is known or is the one token that the step in flight
        is sampling, and the engine takes the step.  Admits waiting requests (as ``plan``
        would); changes nothing else."""
        eng = self.engine
        if not hasattr(eng, "can_queue_ahead"):
            return None
        self._admit()
        if not self.running:
            return None
        entries, blocked = self._try_plan()
        if blocked is not None or not entries:
            return None
        in_flight = {id(r) for r, _ in self._in_flight[1]} if self._in_flight else set()
        shaped = []
        for pe in entries:
            toks = pe.request.all_tokens()[pe.start:pe.start + pe.count]
            if PENDING in toks and not (pe.count == 1 and id(pe.request) in in_flight):
                return None
            shaped.append(StepEntry(self._key(pe.request), [0] * pe.count, [pe.count - 1] if pe.wants_logits else []))
        return entries if eng.can_queue_ahead(shaped) else None

    def _queue_plan(self, planned: List[PlannedEntry]) -> List[tuple]:
        """Queue a planned step (portions of prompts, decode tokens), then take in the ids
        of the step before."""
        from .graph import TokenRef
        before = self._in_flight
        place_before = {id(r): i for i, (r, _) in enumerate(before[1])} if before else {}
        entries, temps, us, wanting = [], [], [], []
        for pe in planned:
            r = pe.request
            toks = r.all_tokens()[pe.start:pe.start + pe.count]
            if pe.count == 1 and toks[0] == PENDING:
                toks = [TokenRef(before[0], place_before[id(r)])]
            entries.append(StepEntry(self._key(r), toks, [pe.count - 1] if pe.wants_logits else []))
            if pe.wants_logits:
                wanting.append(pe)
                temps.append(r.temperature)
                us.append(uniform(r.seed, len(r.generated)))
        try:
            handle = self.engine.step_sample_ahead(entries, temps, us)
        except Exception as exc:
            self._fail_all([pe.request for pe in planned], exc)
            raise
        self.stats["steps"] += 1
        self.stats["tokens"] += sum(pe.count for pe in planned)
        self.stats["max_batch_seen"] = max(self.stats["max_batch_seen"], len(planned))
        for pe in planned:
            key = "decode_tokens" if (pe.count == 1 and pe.request.generated) else "prefill_tokens"
            self.stats[key] += pe.count
            pe.request.cursor += pe.count
        places = []
        for pe in wanting:
            r = pe.request
            places.append((r, len(r.generated)))
            r.generated.append(PENDING)
            if len(r.generated) >= r.max_new_tokens:
                self.running.remove(r)           # its last token is on its way; it takes no further step
        self._in_flight = (handle, places)
        return self._take_in(before) if before else []

    def _queue_ahead(self, requests: List[Request]) -> List[tuple]:
        """Queue one decode token for each of ``requests``, then take in the
        ids of the step before."""
        from .graph import TokenRef
        before = self._in_flight
        place_before = {id(r): i for i, (r, _) in enumerate(before[1])} if before else {}
        entries, temps, us = [], [], []
        for r in requests:
            last = r.generated[-1]
            tok = TokenRef(before[0], place_before[id(r)]) if last == PENDING else last
            entries.append(StepEntry(self._key(r), [tok], [0]))
            temps.append(r.temperature)
            us.append(uniform(r.seed, len(r.generated)))
        try:
            handle = self.engine.step_sample_ahead(entries, temps, us)
        except Exception as exc:
            self._fail_all(requests, exc)
            raise
        self.stats["steps"] += 1
        self.stats["tokens"] += len(requests)
        self.stats["decode_tokens"] += len(requests)
        self.stats["max_batch_seen"] = max(self.stats["max_batch_seen"], len(requests))
        places = []
        for r in requests:
            r.cursor += 1
            places.append((r, len(r.generated)))
            r.generated.append(PENDING)
            if len(r.generated) >= r.max_new_tokens:
                self.running.remove(r)           # its last token is on its way; it takes no further step
        self._in_flight = (handle, places)
        return self._take_in(before) if before else []

    def _take_in(self, flight) -> List[tuple]:
        """Wait for a queued step and book its ids."""
        handle, places = flight
        toks = handle.tokens()
        eos = set(getattr(self.engine, "eos_token_ids", ()) or ())
        newer = {id(r) for r, _ in self._in_flight[1]} if self._in_flight and self._in_flight is not flight else set()
        produced = []
        for (r, at), tok in zip(places, toks):
            if r.overrun:                        # it had ended already: this step was one too many
                del r.generated[at:]
                self.engine.release(self._key(r))
                continue
            r.generated[at] = int(tok)
            produced.append((r.id, int(tok)))
            if r.on_token is not None:
                r.on_token(r.id, int(tok))
            if int(tok) in eos or at + 1 >= r.max_new_tokens:
                r.done = True
                if r in self.running:
                    self.running.remove(r)
                if id(r) in newer:
                    r.overrun = True             # pages go back when the newer step is over
                else:
                    self.engine.release(self._key(r))
        return produced

    def _settle(self) -> List[tuple]:
        """Take in whatever is in flight."""
        flight, self._in_flight = self._in_flight, None
        return self._take_in(flight) if flight else []

    def _fail_all(self, requests, exc):
        try:
            self._settle()
        except Exception:
            self._in_flight = None
        for r in requests:
            r.done, r.error = True, f"step failed: {exc}"
            if self._key(r) in self.engine.cache:
                self.engine.release(self._key(r))
            if r in self.running:
                self.running.remove(r)

    def has_work(self) -> bool:
        return bool(self.running or self.waiting or self._in_flight)

    def run_until_done(self, max_steps: int = 10_000_000) -> Dict[int, Request]:
        steps = 0
        while self.has_work():
            tokens_before = self.stats["tokens"]
            n_before = len(self.running) + len(self.waiting) + (self._in_flight is not None)
            self.step()
            steps += 1
            if (self.stats["tokens"] == tokens_before
                    and len(self.running) + len(self.waiting) + (self._in_flight is not None) == n_before):
                raise SchedulerError("scheduler stands still: no request can take a step")
            if steps > max_steps:
                raise SchedulerError("scheduler did not finish")
        return self.requests

    def stop(self):
        """Fail everything in flight and give its pages back
        (engine/scheduler.go:130-134)."""
        try:
            self._settle()                       # the device is done with the pages after this
        except Exception:
            self._in_flight = None
        for r in list(self.running):
            r.done, r.error = True, "scheduler stopped"
            self.engine.release(self._key(r))
        self.running.clear()
        for r in self.waiting:
            r.done, r.error = True, "scheduler stopped"
        self.waiting.clear()
