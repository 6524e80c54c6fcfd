"""Traces for the replay tests: the same requests cut into steps in four ways.

A trace is a list of steps ``{"step", "entries": [{"id", "tokens", "want"}],
"end"}``, the format ``bin/trace_run`` reads.  Every family asks for the
logits at every position, so each can be compared with the plain
implementation's whole-sequence logits row by row.
"""

import random


def _round64(n):
    return -(-n // 64) * 64


def whole(requests):
    """Each request alone and whole, one step each."""
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
             "end": [rid]} for i, (rid, toks) in enumerate(requests.items())]


def bulk_then_tail(requests, tail=32):
    """All but the last ``tail`` tokens in one step, then one token per step."""
    steps = []
    for rid, toks in requests.items():
        cut = max(1, len(toks) - tail)
        steps.append({"entries": [{"id": rid, "tokens": toks[:cut], "want": list(range(cut))}], "end": []})
        for t in toks[cut:]:
            steps.append({"entries": [{"id": rid, "tokens": [t], "want": [0]}], "end": []})
        steps[-1]["end"] = [rid]
    for i, s in enumerate(steps):
        s["step"] = i
    return steps


def portions(requests, seed=0, sizes=(7, 2, 19, 3, 2, 31, 5, 2, 64, 11)):
    """One request at a time, in portions of changing size, down to two tokens."""
    rng = random.Random(seed)
    steps = []
    for rid, toks in requests.items():
        pos, k = 0, rng.randrange(len(sizes))
        while pos < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - pos)
            k += 1
            steps.append({"entries": [{"id": rid, "tokens": toks[pos:pos + n], "want": list(range(n))}],
                          "end": []})
            pos += n
        steps[-1]["end"] = [rid]
    for i, s in enumerate(steps):
        s["step"] = i
    return steps


def mixed(requests, seed=0, max_live=4, tail=12, max_portion=24):
    """Up to ``max_live`` requests at a time: portions of some beside single
    tokens of others; a request may sit a step out; requests end while others
    go on and new ones start on the pages they gave back.  Returns (steps,
    peak) where peak is the most tokens live requests hold at any time, each
    request's count rounded up to 64: the pool size to replay with."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live = {}                                  # rid -> [tokens, fed]
    steps, peak = [], 0
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
        entries, end = [], []
        for rid, (toks, fed) in list(live.items()):
            if len(live) > 1 and rng.random() < 0.2:
                continue                       # sits this step out
            left = len(toks) - fed
            if left > tail and left - tail >= 2:
                n = min(rng.randint(2, max_portion), left - tail)
            else:
                n = 1
            entries.append({"id": rid, "tokens": toks[fed:fed + n], "want": list(range(n))})
            live[rid][1] = fed + n
        if not entries:
            continue
        peak = max(peak, sum(_round64(f) for _, f in live.values()))
        for rid, (toks, fed) in list(live.items()):
            if fed == len(toks):
                end.append(rid)
                del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps, peak


def peak_tokens(steps):
    held, peak = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(_round64(n) for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak


def collect(steps, outputs):
    """{(request, position): logits row} from per-step outputs ([wanted, vocab]
    arrays or None), in the order of entries and of ``want``."""
    fed, rows = {}, {}
    for s, out in zip(steps, outputs):
        r = 0
        for e in s["entries"]:
            base = fed.get(e["id"], 0)
            for w in e["want"]:
                rows[(e["id"], base + w)] = out[r]
                r += 1
            fed[e["id"]] = base + len(e["tokens"])
        assert (out is None and r == 0) or r == len(out)
    return rows
