"""Builds replay traces (lists of steps in trace_run's JSON form) for the ways of cutting
requests that the tests compare: whole; most in one step and the last 32 tokens one by one;
portions of changing size; and mixed, several live requests with portions beside single
tokens.  Also runs a trace through a ModelRunner and collects logits by (request, position)."""
import random

import torch

from jax_llm_examples_amd.engine import StepEntry

PORTIONS = [7, 2, 13, 3, 2, 29, 5, 2, 17, 31, 2, 3]


def whole(requests):
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
                      "end": [rid]})
    return steps


def tail(requests, last=32):
    steps = []
    for rid, toks in requests.items():
        head = max(0, len(toks) - last)
        cuts = ([(0, head)] if head else []) + [(i, i + 1) for i in range(head, len(toks))]
        for j, (a, b) in enumerate(cuts):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[a:b],
                                                           "want": list(range(b - a))}],
                          "end": [rid] if j == len(cuts) - 1 else []})
    return steps


def portions(requests, sizes=PORTIONS):
    steps = []
    k = 0
    for rid, toks in requests.items():
        o = 0
        while o < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - o)
            k += 1
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[o:o + n],
                                                           "want": list(range(n))}],
                          "end": [rid] if o + n == len(toks) else []})
            o += n
    return steps


def mixed(requests, seed=0, max_live=4, decode_tail=24, max_portion=19):
    """Up to ``max_live`` requests at a time; each step takes from every live request either a
    portion (2..``max_portion`` tokens) or, in its last ``decode_tail`` tokens, one token; now and
    then a request sits a step out."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
        entries, end = [], []
        for rid in list(live):
            toks, o = live[rid]
            if len(live) > 1 and rng.random() < 0.15:
                continue
            left = len(toks) - o
            n = 1 if left <= decode_tail else min(rng.randint(2, max_portion), left - decode_tail)
            entries.append({"id": rid, "tokens": toks[o:o + n], "want": list(range(n))})
            live[rid][1] = o + n
            if o + n == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def max_live_tokens(steps, round_to=64):
    """Most tokens live requests hold at any time, each rounded up to ``round_to``."""
    held, best = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        best = max(best, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return best


def run_trace(runner, steps, record_routing=False):
    """Returns ``{rid: logits [T, V]}`` (and ``{rid: {layer: ids [T, k]}}`` if routing is recorded)."""
    rows, routes, done = {}, {}, {}
    layer_of = {id(b.feed_forward): li for li, b in enumerate(runner.model.blocks)}
    for s in steps:
        entries = [StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]]
        starts = {e.rid: (runner.cache.num_tokens(e.rid) if runner.cache.has_request(e.rid) else 0) for e in entries}
        seen = {}

        def tap(part, name, value):  # the step's parts hand out what they chose
            if name == "routing":
                seen[layer_of[id(part)]] = value[0].clone()

        logits = runner.step(entries, tap=tap if record_routing else None).float().cpu()
        o = t0 = 0
        for e in entries:
            for w in e.want:
                rows.setdefault(e.rid, {})[starts[e.rid] + w] = logits[o]
                o += 1
            for li, ids in seen.items():
                routes.setdefault(e.rid, {}).setdefault(li, []).append(ids[t0:t0 + len(e.tokens)].cpu())
            t0 += len(e.tokens)
        for rid in s["end"]:
            runner.finish(rid)
    out = {rid: torch.stack([r[i] for i in range(len(r))]) for rid, r in rows.items()}
    if record_routing:
        return out, {rid: {li: torch.cat(v) for li, v in d.items()} for rid, d in routes.items()}
    return out


def random_requests(vocab, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}
