"""Ways of cutting the same requests into steps: whole, most of it at once and the last 32 one
by one, portions of changing size, and mixed (several live requests, portions beside single
tokens, requests ending and starting so that pages are used again).

A trace is a list of steps {"step": n, "entries": [{"id", "tokens", "want"}], "end": [...]}, the
format bin/trace_run reads.  Logits are wanted at every fed position unless `want_every` is
larger than 1."""
from __future__ import annotations

import random


def _entry(rid, tokens, start, n, want_every=1):
    want = [i for i in range(n) if (start + i) % want_every == 0 or start + i == len(tokens) - 1]
    return {"id": rid, "tokens": tokens[start:start + n], "want": want}


def whole(requests, want_every=1):
    """Every request alone, all its tokens in one step."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [_entry(rid, toks, 0, len(toks), want_every)], "end": [rid]})
    return steps


def tail_singly(requests, tail=32, want_every=1):
    """Most of a request in one step, its last `tail` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(0, len(toks) - tail)
        if head:
            steps.append({"step": len(steps), "entries": [_entry(rid, toks, 0, head, want_every)], "end": []})
        for p in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [_entry(rid, toks, p, 1, want_every)], "end": [rid] if p == len(toks) - 1 else []})
    return steps


def portions(requests, sizes=(7, 2, 5, 3, 2, 11, 1, 4), want_every=1):
    """Each request alone, cut into portions whose sizes cycle through `sizes` (down to two tokens and one)."""
    steps = []
    for k, (rid, toks) in enumerate(requests.items()):
        p, i = 0, k                      # every request starts elsewhere in the cycle
        while p < len(toks):
            n = min(sizes[i % len(sizes)], len(toks) - p)
            steps.append({"step": len(steps), "entries": [_entry(rid, toks, p, n, want_every)], "end": [rid] if p + n == len(toks) else []})
            p, i = p + n, i + 1
    return steps


def mixed(requests, seed=0, max_live=4, prompt_share=0.6, portion=(2, 9), want_every=1):
    """Up to `max_live` requests at a time.  The first `prompt_share` of a request is fed in portions
    of portion[0]..portion[1] tokens (2..9 unless said otherwise), the rest one token a step; in every step a random
    non-empty subset of the live requests takes part; a finished request ends and the next one starts."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live, fed, steps = [], {}, []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            rid, toks = waiting.pop(0)
            live.append(rid)
            fed[rid] = 0
        part = [r for r in live if rng.random() < 0.75] or [rng.choice(live)]
        entries, ended = [], []
        for rid in part:
            toks = requests[rid]
            prompt = max(1, int(len(toks) * prompt_share))
            n = min(rng.randint(*portion), prompt - fed[rid]) if fed[rid] < prompt else 1
            entries.append(_entry(rid, toks, fed[rid], n, want_every))
            fed[rid] += n
            if fed[rid] == len(toks):
                ended.append(rid)
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        for rid in ended:
            live.remove(rid)
    return steps


def peak_tokens(steps, round_to=64):
    """Most tokens live requests hold at any time, each request rounded up to a multiple of `round_to`."""
    held, peak = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak


def wanted_positions(steps):
    """For every step with wanted logits: the (request, position) of each row written, in order."""
    fed, out = {}, {}
    for s in steps:
        rows = []
        for e in s["entries"]:
            start = fed.get(e["id"], 0)
            rows += [(e["id"], start + w) for w in e["want"]]
            fed[e["id"]] = start + len(e["tokens"])
        for rid in s["end"]:
            fed.pop(rid, None)
        if rows:
            out[s["step"]] = rows
    return out
