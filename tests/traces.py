"""Builders of replay traces (the JSON steps bin/trace_run reads) for the four cuttings,
and the bookkeeping that says which (request, position) each written logits row is."""
import random
from typing import Dict, List, Sequence, Tuple


def _step(n, entries, end=()):
    return {"step": n, "entries": entries, "end": list(end)}


def whole(requests: Dict[str, Sequence[int]]):
    """Each request alone and whole: one step per request, every position wanted."""
    steps = []
    for i, (rid, toks) in enumerate(requests.items()):
        steps.append(_step(i, [{"id": rid, "tokens": list(toks), "want": list(range(len(toks)))}], [rid]))
    return steps


def tail_one_by_one(requests: Dict[str, Sequence[int]], tail: int = 32):
    """Most of a request in one step, the last `tail` tokens one by one."""
    steps = []
    n = 0
    for rid, toks in requests.items():
        toks = list(toks)
        head = max(1, len(toks) - tail)
        steps.append(_step(n, [{"id": rid, "tokens": toks[:head], "want": list(range(head))}]))
        n += 1
        for i in range(head, len(toks)):
            steps.append(_step(n, [{"id": rid, "tokens": [toks[i]], "want": [0]}], [rid] if i == len(toks) - 1 else []))
            n += 1
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests: Dict[str, Sequence[int]], sizes=(7, 2, 19, 3, 2, 33, 5, 2, 16, 1, 64, 2, 9)):
    """Portions of changing size, down to two tokens, at odd offsets across page edges."""
    steps = []
    n = 0
    k = 0
    for rid, toks in requests.items():
        toks = list(toks)
        at = 0
        while at < len(toks):
            m = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            last = at + m == len(toks)
            steps.append(_step(n, [{"id": rid, "tokens": toks[at:at + m], "want": list(range(m))}], [rid] if last else []))
            n += 1
            at += m
    return steps


def mixed(requests: Dict[str, Sequence[int]], seed: int = 0, max_live: int = 4, decode_tail: int = 12):
    """Up to `max_live` live requests; each step holds portions of some beside single decoded
    tokens of others; a request is sometimes left out of a step.  Returns (steps, max_tokens)
    where max_tokens is the most that live requests hold at any time, each rounded up to 64."""
    rng = random.Random(seed)
    waiting = [(rid, list(t)) for rid, t in requests.items()]
    live: List[Tuple[str, List[int]]] = []
    done_at: Dict[str, int] = {}
    steps = []
    n = 0
    peak = 0
    r64 = lambda x: -(-x // 64) * 64
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live.append((rid, toks))
            done_at[rid] = 0
        entries, ended = [], []
        for rid, toks in live:
            at = done_at[rid]
            left = len(toks) - at
            if len(live) > 1 and rng.random() < 0.2 and entries:
                continue                                  # left out of this step, goes on later
            if left <= decode_tail:
                m = 1
            else:
                m = min(left - decode_tail, rng.choice([2, 3, 5, 8, 13, 21, 30]))
            entries.append({"id": rid, "tokens": toks[at:at + m], "want": list(range(m))})
            done_at[rid] = at + m
            if at + m == len(toks):
                ended.append(rid)
        peak = max(peak, sum(r64(done_at[rid]) for rid, _ in live))
        if entries:
            steps.append(_step(n, entries, ended))
            n += 1
        live = [(rid, t) for rid, t in live if rid not in ended]
    return steps, peak


def rows_of(steps) -> Dict[int, List[Tuple[str, int]]]:
    """For each step that writes a file: the (request, position) of every row, in order."""
    at: Dict[str, int] = {}
    out = {}
    for s in steps:
        rows = []
        for e in s["entries"]:
            base = at.get(e["id"], 0)
            rows += [(e["id"], base + w) for w in e.get("want", [])]
            at[e["id"]] = base + len(e["tokens"])
        for rid in s["end"]:
            at.pop(rid, None)
        if rows:
            out[s["step"]] = rows
    return out
