"""The scheduler's decisions, with a stand-in for the engine (no GPU): the
stand-in keeps a real cache manager and answers every wanted place with
logits that are a fixed function of the request's tokens up to that place."""

import random

import pytest

from kllm_amd.cache import CacheManager, GroupSpec, OutOfPages
from kllm_amd.engine.scheduler import Scheduler, SchedulerError
from kllm_amd.sampling import sample_host, uniform

V = 50


def next_token(prefix):
    h = 7
    for t in prefix:
        h = (h * 31 + t + 1) % 1000003
    return h % V


class StandIn:
    def __init__(self, num_pages=64, page_size=4, slots=16, eos=(), max_model_len=None, window=0):
        self.cache = CacheManager([GroupSpec("g", page_size, num_pages, window)], slots)
        self.seen = {}                 # request -> tokens in its cache
        self.eos_token_ids = tuple(eos)
        self.max_model_len = max_model_len
        self.steps = []                # per step: list of (request, count)

    def step(self, entries):
        for e in entries:
            self.cache.reserve(e.request_id, len(e.tokens))   # raises OutOfPages like the engine
        rows = []
        for e in entries:
            have = self.seen.setdefault(e.request_id, [])
            assert len(have) == self.cache.get(e.request_id).length
            for w in e.want:
                row = [0.0] * V
                row[next_token(have + list(e.tokens[:w + 1]))] = 5.0
                rows.append(row)
            have.extend(e.tokens)
            self.cache.commit(e.request_id, len(e.tokens))
        self.steps.append([(e.request_id, len(e.tokens)) for e in entries])
        self.cache.check_invariants()
        return rows

    def sample(self, logits, temps, us):
        return sample_host(logits, temps, us)

    def release(self, rid):
        self.seen.pop(rid, None)
        self.cache.release(rid)


def alone(prompt, n, eos=()):
    toks, out = list(prompt), []
    for _ in range(n):
        t = next_token(toks)
        out.append(t)
        toks.append(t)
        if t in eos:
            break
    return out


def prompts(seed, count, lo=1, hi=40):
    rng = random.Random(seed)
    return [[rng.randrange(V) for _ in range(rng.randint(lo, hi))] for _ in range(count)]


def test_every_request_gets_its_tokens_whatever_the_batching():
    ps = prompts(1, 9)
    eng = StandIn()
    s = Scheduler(eng, max_batch=4, max_step_tokens=16)
    ids = [s.submit(p, 12) for p in ps]
    res = s.run_until_done()
    for i, p in zip(ids, ps):
        assert res[i].tokens == alone(p, 12) and res[i].done and res[i].error is None
    assert eng.cache.pools[0].free_pages == 64 and eng.cache.slots.free_slots == 16
    assert s.stats["max_batch_seen"] == 4            # queueing happened, batches were mixed


def test_token_budget_and_portions():
    ps = prompts(2, 6, lo=20, hi=70)
    eng = StandIn(num_pages=200)
    s = Scheduler(eng, max_batch=3, max_step_tokens=24, chunk_size=10)
    ids = [s.submit(p, 5) for p in ps]
    res = s.run_until_done()
    fed = {}
    for step in eng.steps:
        assert sum(c for _, c in step) <= 24                       # budget never exceeded
        assert len(step) <= 3
        for rid, c in step:
            fed[rid] = fed.get(rid, 0) + c
            assert c <= 10 or c == 1
    for i, p in zip(ids, ps):
        assert res[i].tokens == alone(p, 5)
        assert fed[s._key(res[i])] == len(p) + 4                   # portions sum to the prompt
    # decoding requests go first: once a request decodes, every later step holds it
    first_decode = {}
    for n, step in enumerate(eng.steps):
        for rid, c in step:
            if c == 1 and rid not in first_decode and fed[rid] > 1:
                first_decode[rid] = n
    assert s.stats["prefill_tokens"] == sum(len(p) for p in ps)
    assert s.stats["decode_tokens"] == 4 * len(ps)


def test_steps_end_on_whole_tiles_of_rows():
    """With an engine whose products work on tiles of 8 rows, a step of more
    than one tile that ends less than half a tile above a multiple gives the
    excess of its last prompt portion back; everything else stays as planned,
    and every request still gets its tokens."""
    ps = prompts(5, 6, lo=30, hi=90)
    plain, trimmed = StandIn(num_pages=400), StandIn(num_pages=400)
    trimmed.step_row_multiple = 8
    outs = []
    for eng in (plain, trimmed):
        s = Scheduler(eng, max_batch=4, max_step_tokens=35, chunk_size=32)
        assert s.row_multiple == (8 if eng is trimmed else 0)
        ids = [s.submit(p, 6) for p in ps]
        res = s.run_until_done()
        outs.append([res[i].tokens for i in ids])
        assert s.stats["prefill_tokens"] == sum(len(p) for p in ps)
    assert outs[0] == outs[1] == [alone(p, 6) for p in ps]
    sizes = [sum(c for _, c in step) for step in plain.steps]
    assert any(t > 8 and 0 < t % 8 < 4 for t in sizes)              # the plain plan has such steps
    for step in trimmed.steps:
        total = sum(c for _, c in step)
        last_is_prompt = step[-1][1] > 1
        if total > 8 and last_is_prompt:
            assert not 0 < total % 8 < 4, step
    assert Scheduler(plain, row_multiple=16).row_multiple == 16     # the caller may say it


def test_stops_at_eos_and_at_the_limit():
    p = [3, 1, 4, 1, 5]
    free_run = alone(p, 30)
    eos = free_run[6]
    cut = free_run.index(eos) + 1
    eng = StandIn(eos=(eos,))
    s = Scheduler(eng)
    i = s.submit(p, 30)
    j = s.submit(p, 3)
    res = s.run_until_done()
    assert res[i].tokens == free_run[:cut] and res[i].tokens[-1] == eos    # the EOS token is emitted
    assert res[j].tokens == alone(p, 3, eos=(eos,))
    assert eng.cache.pools[0].free_pages == 64


def test_what_can_never_run_is_refused_at_submit():
    eng = StandIn(num_pages=4, page_size=4, max_model_len=100)
    s = Scheduler(eng)
    with pytest.raises(SchedulerError):
        s.submit([], 4)
    with pytest.raises(SchedulerError):
        s.submit([1], 0)
    with pytest.raises(SchedulerError, match="pages"):
        s.submit([1] * 10, 8)                        # 18 tokens need 5 pages, the pool has 4
    with pytest.raises(SchedulerError, match="longest"):
        s.submit([1] * 90, 11)
    s.submit([1] * 10, 6)                            # 16 tokens fit exactly


def test_a_long_request_fits_a_windowed_pool_when_its_portions_are_small():
    """A windowed group holds the window and one portion, not the request: 200 tokens
    run in a pool of 6 pages of 4 when no step brings more than 8, and are refused at
    submit when a step may bring them all."""
    p = prompts(3, 1, lo=150, hi=150)[0]
    eng = StandIn(num_pages=6, page_size=4, window=9)
    with pytest.raises(SchedulerError, match="could not run even alone"):
        Scheduler(eng, max_batch=2, max_step_tokens=2048).submit(p, 50)
    s = Scheduler(eng, max_batch=2, max_step_tokens=8)
    i = s.submit(p, 50)
    res = s.run_until_done()
    assert res[i].tokens == alone(p, 50) and res[i].error is None
    assert eng.cache.pools[0].high_water <= 6 and eng.cache.pools[0].free_pages == 6


def test_long_prompt_is_cut_not_refused():
    # the reference refuses a prompt longer than the step budget (engine/scheduler.go:64-70)
    eng = StandIn(num_pages=100)
    s = Scheduler(eng, max_step_tokens=8)
    p = prompts(3, 1, lo=50, hi=50)[0]
    i = s.submit(p, 4)
    assert s.run_until_done()[i].tokens == alone(p, 4)
    assert max(sum(c for _, c in st) for st in eng.steps) == 8


def test_preemption_under_a_tiny_pool_changes_no_token():
    ps = prompts(4, 6, lo=5, hi=14)
    eng = StandIn(num_pages=9, page_size=4)          # 36 tokens of cache for six requests
    s = Scheduler(eng, max_batch=4, max_step_tokens=32)
    ids = [s.submit(p, 16) for p in ps]
    res = s.run_until_done()
    for i, p in zip(ids, ps):
        assert res[i].tokens == alone(p, 16), i
    assert s.stats["preemptions"] > 0
    assert sum(r.preemptions for r in res.values()) == s.stats["preemptions"]
    assert eng.cache.pools[0].free_pages == 9 and eng.cache.slots.free_slots == 16
    # the youngest goes first: request 0 is never preempted
    assert res[ids[0]].preemptions == 0


def test_the_plan_never_overdraws_the_pool():
    rng = random.Random(5)
    for trial in range(20):
        eng = StandIn(num_pages=rng.randint(6, 20), page_size=rng.choice([2, 4, 8]))
        s = Scheduler(eng, max_batch=rng.randint(1, 5), max_step_tokens=rng.randint(4, 40),
                      chunk_size=rng.randint(2, 40))
        cap = eng.cache.pools[0].num_pages * eng.cache.groups[0].page_size
        ps = [p for p in prompts(trial, 7, hi=25) if len(p) + 6 <= cap]
        ids = [s.submit(p, 6) for p in ps]
        res = s.run_until_done()              # StandIn.step raises OutOfPages if a plan overdraws
        for i, p in zip(ids, ps):
            assert res[i].tokens == alone(p, 6)


def test_temperature_uses_one_uniform_per_generated_token():
    class Spy(StandIn):
        def sample(self, logits, temps, us):
            self.calls.append((list(temps), list(us)))
            return super().sample(logits, temps, us)
    eng = Spy()
    eng.calls = []
    s = Scheduler(eng, max_batch=2)
    a = s.submit([1, 2, 3], 3, temperature=0.8, seed=11)
    b = s.submit([4, 5], 3, temperature=0.0, seed=12)
    s.run_until_done()
    seen = {11: [], 12: []}
    for temps, us in eng.calls:
        for t, u in zip(temps, us):
            seen[11 if t == 0.8 else 12].append(u)
    assert seen[11] == [uniform(11, k) for k in range(3)]
    assert seen[12] == [uniform(12, k) for k in range(3)]


def test_stop_fails_what_is_in_flight():
    eng = StandIn()
    s = Scheduler(eng, max_batch=1)
    a, b = s.submit([1, 2, 3], 50), s.submit([4], 5)
    s.step(), s.step()
    s.stop()
    assert s.requests[a].error == "scheduler stopped" and s.requests[b].error == "scheduler stopped"
    assert eng.cache.pools[0].free_pages == 64 and not s.has_work()


def test_a_failed_step_fails_its_requests():
    class Broken(StandIn):
        def step(self, entries):
            raise RuntimeError("device lost")
    eng = Broken()
    s = Scheduler(eng)
    a = s.submit([1, 2], 4)
    with pytest.raises(RuntimeError):
        s.step()
    assert "device lost" in s.requests[a].error and not s.running
    assert eng.cache.slots.free_slots == 16


# ------------------------------------------------------------------ one step ahead

class FakeHandle:
    """What a queued step returns: its ids exist only after tokens() is called,
    and until then the "device" still works on the step's requests."""

    def __init__(self, engine, compute, rids):
        self.engine, self._compute, self.rids, self._ids = engine, compute, rids, None
        self.count = len(rids)
        engine.in_flight.append(self)

    def tokens(self):
        if self._ids is None:
            self._ids = self._compute()
            self.engine.in_flight.remove(self)
        return self._ids


class StandInAhead(StandIn):
    """A stand-in that can queue a step of decode tokens before the ids of the
    step before are known, as the engine does with its HIP graphs."""

    def __init__(self, *a, **k):
        super().__init__(*a, **k)
        self.in_flight = []
        self.last = None
        self.ahead_steps = 0

    def can_sample_ahead(self, entries):
        return bool(entries) and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries)

    def step_sample_ahead(self, entries, temps, us):
        from kllm_amd.engine.graph import TokenRef
        for e in entries:
            t = e.tokens[0]
            assert not isinstance(t, TokenRef) or t.source is self.last, "a reference to an older step"
        for e in entries:
            self.cache.reserve(e.request_id, 1)
        for e in entries:
            self.cache.commit(e.request_id, 1)      # the engine commits when it queues
        before, refs = self.last, [e.tokens[0] for e in entries]

        def compute():
            out = []
            for e, t in zip(entries, refs):
                tok = before.tokens()[t.index] if isinstance(t, TokenRef) else t
                have = self.seen.setdefault(e.request_id, [])
                have.append(tok)
                out.append(next_token(have))
            return out
        self.steps.append([(e.request_id, 1) for e in entries])
        self.ahead_steps += 1
        self.last = FakeHandle(self, compute, [e.request_id for e in entries])
        return self.last

    def step_sample(self, entries, temps, us):
        assert not self.in_flight, "a plain step while another is in flight"
        rows = self.step(entries)
        return self.sample(rows, temps, us) if rows else []

    def release(self, rid):
        assert all(rid not in h.rids for h in self.in_flight), "pages given back under a running step"
        super().release(rid)


@pytest.mark.parametrize("eos", [(), (7, 21, 33)])
def test_one_step_ahead_gives_the_same_tokens_and_returns_every_page(eos):
    ps = prompts(11, 10, lo=1, hi=30)
    news = [1, 2, 3, 17, 40, 9, 25, 6, 31, 12]
    eng = StandInAhead(num_pages=400, eos=eos)
    s = Scheduler(eng, max_batch=4, max_step_tokens=32)
    seen = {}
    ids = [s.submit(p, n, on_token=lambda i, t: seen.setdefault(i, []).append(t)) for p, n in zip(ps, news)]
    res = s.run_until_done()
    assert eng.ahead_steps > 5 and not eng.in_flight
    for i, p, n in zip(ids, ps, news):
        want = alone(p, n, eos)
        assert res[i].tokens == want and res[i].done and res[i].error is None, (i, res[i].tokens, want)
        assert seen[i] == want                      # callbacks saw every token once, in order
    assert eng.cache.pools[0].free_pages == 400 and eng.cache.slots.free_slots == 16
    eng.cache.check_invariants()


def test_an_end_of_sequence_id_is_seen_one_step_late_and_the_extra_token_dropped():
    p = [3, 1, 4]
    first = alone(p, 50)
    eos_at = 5
    eos = (first[eos_at],)
    assert first[eos_at] not in first[:eos_at]
    eng = StandInAhead(eos=eos)
    s = Scheduler(eng, max_batch=2, max_step_tokens=16)
    i = s.submit(p, 50)
    res = s.run_until_done()
    assert res[i].tokens == first[:eos_at + 1]
    decode_steps = sum(1 for st in eng.steps if st == [(("sched", id(s), i), 1)])
    assert decode_steps == eos_at + 1               # one step more than the tokens after the first
    assert eng.cache.pools[0].free_pages == 64


def test_stop_with_a_step_in_flight():
    eng = StandInAhead()
    s = Scheduler(eng, max_batch=2, max_step_tokens=16)
    i = s.submit([1, 2, 3], 30)
    for _ in range(4):
        s.step()
    assert eng.in_flight
    s.stop()
    assert not eng.in_flight and eng.cache.pools[0].free_pages == 64 and s.requests[i].done
