"""Ways of cutting the same requests into steps, as trace-replay records.

Every function returns a list of step records ({"step", "entries", "end"}); every token's logits are wanted
unless `want_last_only`. `place[(step, row)] = (request, position)` tells which logits row is which.
"""
import numpy as np


def _finish(steps):
    place = {}
    pos = {}
    for rec in steps:
        row = 0
        for e in rec["entries"]:
            start = pos.get(e["id"], 0)
            for w in e["want"]:
                place[(rec["step"], row)] = (e["id"], start + w)
                row += 1
            pos[e["id"]] = start + len(e["tokens"])
        for r in rec["end"]:
            pos.pop(r, None)
    return steps, place


def whole(requests):
    """Each request alone and whole: one step per request."""
    steps = []
    for i, (rid, toks) in enumerate(requests.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": list(toks), "want": list(range(len(toks)))}],
                      "end": [rid]})
    return _finish(steps)


def head_then_singles(requests, tail=32):
    """Most of a request in one step, its last `tail` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        toks = list(toks)
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}],
                      "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}], "end": []})
        steps[-1]["end"] = [rid]
    return _finish(steps)


def portions(requests, sizes=(7, 2, 13, 3, 2, 30, 5, 2, 64, 17, 2, 9)):
    """Portions of changing size, down to two tokens."""
    steps = []
    for rid, toks in requests.items():
        toks = list(toks)
        i, k = 0, 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[i:i + n],
                                                           "want": list(range(n))}], "end": []})
            i += n
        steps[-1]["end"] = [rid]
    return _finish(steps)


def mixed(requests, max_tokens, page=64, seed=0, tail=32, max_live=4):
    """Up to `max_live` live requests: portions of some beside single decoded tokens of others, some
    requests left out of a step, new ones admitted as soon as the page budget (`max_tokens`, each request's
    count rounded up to `page`) allows, so that pages of finished requests are used again."""
    rng = np.random.default_rng(seed)
    waiting = [(rid, list(t)) for rid, t in requests.items()]
    live = {}           # rid -> [tokens, done]
    steps = []

    def rounded(n):
        return -(-n // page) * page

    while waiting or live:
        budget = max_tokens - sum(rounded(len(t)) for t, _ in live.values())
        while waiting and len(live) < max_live and rounded(len(waiting[0][1])) <= budget:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
            budget -= rounded(len(toks))
        if not live:
            raise ValueError("a request does not fit the token budget")
        entries, end = [], []
        chosen = [rid for rid in live if rng.random() < 0.8] or [next(iter(live))]
        for rid in chosen:
            toks, done = live[rid]
            left = len(toks) - done
            if left <= tail:
                n = 1
            else:
                n = int(min(left - tail, rng.integers(2, 40)))
                if left - tail - n == 1:      # never leave a portion of one token before the tail
                    n += 1
            entries.append({"id": rid, "tokens": toks[done:done + n], "want": list(range(n))})
            live[rid][1] = done + n
            if done + n == len(toks):
                end.append(rid)
        for rid in end:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return _finish(steps)


def only_last(made):
    """The same steps with logits wanted at the last token of each request alone: every other entry wants
    nothing, and many a step wants nothing at all."""
    steps, _ = made
    out = []
    for rec in steps:
        entries = [dict(e, want=[len(e["tokens"]) - 1] if e["id"] in rec["end"] else []) for e in rec["entries"]]
        out.append(dict(rec, entries=entries))
    return _finish(out)
